"""CPU oracle for sliding-window 2-simplicial attention.  TEST INFRASTRUCTURE ONLY.

This file is a checker, not a product path: it may be imported by ``tests/``,
by ``__graft_entry__.smoke()`` and by the ``cpu_baseline`` leg of ``bench.py``
and by nothing else.  The shipped operator never routes through it.

It restates, in plain PyTorch (fp32 or fp64, any device, no custom kernels),
the algorithm of the reference:

* ``naive_two_simplicial_attend``  follows simplicial_attention/simplicial_attention.py:78-127
  (scale :102-104, GQA grouping :93-98 and :127, causal mask :111-117,
  joint softmax over the flattened (j, k) plane :119-123, value contraction :125).
* the sliding windows follow the kernel masks of
  simplicial_attention/triton_two_simplicial_attention.py:191-193 and the test
  mask of tests/test_triton.py:33-47:  ``0 <= i - j < w1`` and ``0 <= i - k < w2``.
* ``windowed_dense`` is the dense O(N^3) form of that windowed operator in the
  kernel's ``(b, n, h, d)`` layout; ``windowed_banded`` is the same operator
  evaluated per query chunk over only the rows the windows can reach, so that it
  scales to N = 8192 / 32768.
* ``windowed_grads_explicit`` evaluates the backward formulas that the reference
  kernels implement (triton_two_simplicial_attention.py:282, 478-489, 662-699, 709)
  without autograd, so that autograd through the forward restatement and the
  closed-form gradients pin each other.

Parity status: the reference holds no golden vectors for this path
(tests/test_triton.py compares two GPU implementations at run time).  Every
function here is pinned by tests/test_oracle_pins.py against: brute-force
loops on tiny inputs, torch's scaled_dot_product_attention over the flattened
N^2 key set (the construction of tests/test_triton.py:52-64), closed-form special
cases, invariants, ``torch.autograd.gradcheck`` and the independent fp64 C
restatement in oracle/sa2_oracle.c.
"""
from __future__ import annotations

import math

import torch
from torch import Tensor


# ---------------------------------------------------------------------------
# dense full-causal form in the reference's head-first layout
# ---------------------------------------------------------------------------

def naive_two_simplicial_attend(q: Tensor, k, v, causal: bool = False) -> Tensor:
    """Dense 2-simplicial attention, layout ``b h n d`` (simplicial_attention.py:78-127).

    ``k = (k1, k2)`` and ``v = (v1, v2)`` carry ``kv_heads`` heads; query head
    ``h * g + r`` reads key/value head ``h`` (simplicial_attention.py:98,127).
    """
    assert len(k) == len(v) == 2
    k1, k2 = k
    v1, v2 = v
    b, heads, n, d = q.shape
    kv_heads = k1.shape[1]
    assert heads % kv_heads == 0
    g = heads // kv_heads

    qg = q.reshape(b, kv_heads, g, n, d) * (d ** -0.5)
    sim = torch.einsum('bhgid,bhjd,bhkd->bhgijk', qg, k1, k2)

    if causal:
        nj = sim.shape[-1]
        assert sim.shape[-2] == nj
        upper = torch.ones(n, nj, dtype=torch.bool, device=q.device).triu(nj - n + 1)
        blocked = upper[:, :, None] | upper[:, None, :]
        sim = sim.masked_fill(blocked, -torch.finfo(sim.dtype).max)

    attn = sim.flatten(-2).softmax(dim=-1).reshape(sim.shape)
    out = torch.einsum('bhgijk,bhjd,bhkd->bhgid', attn, v1, v2)
    return out.reshape(b, heads, n, v1.shape[-1])


# ---------------------------------------------------------------------------
# windowed operator, kernel layout (b, n, h, d)
# ---------------------------------------------------------------------------

def window_mask(n: int, w1: int, w2: int, device=None) -> Tensor:
    """Boolean [n, n, n] mask, True where (i, j, k) is attended
    (triton_two_simplicial_attention.py:191-193; tests/test_triton.py:33-47)."""
    idx = torch.arange(n, device=device)
    d = idx[:, None] - idx[None, :]                 # i - j
    m1 = (d >= 0) & (d < w1)
    m2 = (d >= 0) & (d < w2)
    return m1[:, :, None] & m2[:, None, :]


def expand_kv_heads(t: Tensor, groups: int) -> Tensor:
    """'b n h d -> b n (h g) d' (triton_two_simplicial_attention.py:1033-1034)."""
    if groups == 1:
        return t
    return t.repeat_interleave(groups, dim=2)


def windowed_dense(q, k1, k2, v1, v2, w1: int, w2: int, scale: float | None = None):
    """Dense windowed 2-simplicial attention.  All tensors ``(b, n, h, d)`` with
    equal head counts.  Returns ``(out [b n h d], lse [b h n])`` where ``lse`` is
    the natural-log normaliser the reference saves as ``M``
    (triton_two_simplicial_attention.py:225-228)."""
    b, n, h, d = q.shape
    scale = d ** -0.5 if scale is None else scale
    sim = torch.einsum('bihd,bjhd,bkhd->bhijk', q, k1, k2) * scale
    allowed = window_mask(n, w1, w2, q.device)
    sim = sim.masked_fill(~allowed, float('-inf'))
    flat = sim.flatten(-2)
    lse = torch.logsumexp(flat, dim=-1)
    attn = torch.exp(flat - lse[..., None]).reshape(sim.shape)
    out = torch.einsum('bhijk,bjhd,bkhd->bihd', attn, v1, v2)
    return out, lse


def _banded_chunk(q, k1, k2, v1, v2, i0, i1, w1, w2, scale):
    """Rows [i0, i1) of the windowed operator using only reachable key rows."""
    j0 = max(0, i0 - w1 + 1)
    k0 = max(0, i0 - w2 + 1)
    qi = q[:, i0:i1]
    a1, b1 = k1[:, j0:i1], v1[:, j0:i1]
    a2, b2 = k2[:, k0:i1], v2[:, k0:i1]
    sim = torch.einsum('bihd,bjhd,bkhd->bhijk', qi, a1, a2) * scale
    ii = torch.arange(i0, i1, device=q.device)
    jj = torch.arange(j0, i1, device=q.device)
    kk = torch.arange(k0, i1, device=q.device)
    dj = ii[:, None] - jj[None, :]
    dk = ii[:, None] - kk[None, :]
    allowed = ((dj >= 0) & (dj < w1))[:, :, None] & ((dk >= 0) & (dk < w2))[:, None, :]
    sim = sim.masked_fill(~allowed, float('-inf'))
    flat = sim.flatten(-2)
    lse = torch.logsumexp(flat, dim=-1)
    attn = torch.exp(flat - lse[..., None]).reshape(sim.shape)
    out = torch.einsum('bhijk,bjhd,bkhd->bihd', attn, b1, b2)
    return out, lse


def windowed_banded(q, k1, k2, v1, v2, w1: int, w2: int, scale: float | None = None,
                    chunk: int = 64):
    """Same operator as :func:`windowed_dense`, evaluated in query chunks over the
    band only: O(N * (w1 + chunk) * (w2 + chunk) * D) time, O(chunk * w1 * w2)
    memory.  Differentiable by autograd."""
    b, n, h, d = q.shape
    scale = d ** -0.5 if scale is None else scale
    outs, lses = [], []
    for i0 in range(0, n, chunk):
        o, l = _banded_chunk(q, k1, k2, v1, v2, i0, min(n, i0 + chunk), w1, w2, scale)
        outs.append(o)
        lses.append(l)
    return torch.cat(outs, dim=1), torch.cat(lses, dim=-1)


def windowed_banded_fwd_bwd(q, k1, k2, v1, v2, dout, w1, w2, scale=None, chunk: int = 64):
    """Forward and all five input gradients of the banded operator for the loss
    ``(out * dout).sum()``; autograd is run chunk by chunk so that memory stays
    O(chunk * w1 * w2).  Returns ``out, lse, (dq, dk1, dk2, dv1, dv2)``."""
    b, n, h, d = q.shape
    scale = d ** -0.5 if scale is None else scale
    leaves = [t.detach().clone().requires_grad_(True) for t in (q, k1, k2, v1, v2)]
    outs, lses = [], []
    for i0 in range(0, n, chunk):
        i1 = min(n, i0 + chunk)
        o, l = _banded_chunk(*leaves, i0, i1, w1, w2, scale)
        (o * dout[:, i0:i1]).sum().backward()
        outs.append(o.detach())
        lses.append(l.detach())
    grads = tuple(t.grad for t in leaves)
    return torch.cat(outs, dim=1), torch.cat(lses, dim=-1), grads


def windowed_grads_explicit(q, k1, k2, v1, v2, dout, w1: int, w2: int, scale: float | None = None):
    """Closed-form gradients of the dense windowed operator, no autograd.

    delta = rowsum(o * do)              triton_two_simplicial_attention.py:282
    dp    = do . (v1_j * v2_k)          :481, :686
    ds    = p * (dp - delta)            :482, :687
    dv1   = sum_{i,k} p  do v2          :478-479        dv2 = sum_{i,j} p  do v1   :680-683
    dk1   = scale sum_{i,k} ds q k2     :487-489        dk2 = scale sum_{i,j} ds q k1  :662,695
    dq    = scale sum_{j,k} ds k1 k2    :697-699, 709
    """
    b, n, h, d = q.shape
    scale = d ** -0.5 if scale is None else scale
    out, lse = windowed_dense(q, k1, k2, v1, v2, w1, w2, scale)
    sim = torch.einsum('bihd,bjhd,bkhd->bhijk', q, k1, k2) * scale
    allowed = window_mask(n, w1, w2, q.device)
    p = torch.exp(sim - lse[..., None, None]).masked_fill(~allowed, 0.0)
    delta = (out * dout).sum(-1).permute(0, 2, 1)                       # b h i
    dp = torch.einsum('bihd,bjhd,bkhd->bhijk', dout, v1, v2)
    ds = p * (dp - delta[..., None, None])
    dv1 = torch.einsum('bhijk,bihd,bkhd->bjhd', p, dout, v2)
    dv2 = torch.einsum('bhijk,bihd,bjhd->bkhd', p, dout, v1)
    dk1 = torch.einsum('bhijk,bihd,bkhd->bjhd', ds, q, k2) * scale
    dk2 = torch.einsum('bhijk,bihd,bjhd->bkhd', ds, q, k1) * scale
    dq = torch.einsum('bhijk,bjhd,bkhd->bihd', ds, k1, k2) * scale
    return out, lse, delta, (dq, dk1, dk2, dv1, dv2)


def sliding_two_simplicial_attn(q, keys, values, w1=512, w2=32, causal=True,
                                pad_to_multiple_of=64, dense: bool | None = None):
    """Oracle counterpart of the functional wrapper
    (triton_two_simplicial_attention.py:1020-1056): GQA expansion in ``(h g)``
    order, zero right-padding of the sequence and slicing back.  Padding rows sit
    after every real row, so under the causal windows they cannot influence real
    rows; the pad/slice is still carried out literally here."""
    assert causal, 'the reference only defines the causal operator (triton_two_simplicial_attention.py:1073)'
    hq, hk = q.shape[-2], keys[0].shape[-2]
    assert hq % hk == 0
    g = hq // hk
    k1, k2 = (expand_kv_heads(t, g) for t in keys)
    v1, v2 = (expand_kv_heads(t, g) for t in values)
    n = q.shape[1]
    if pad_to_multiple_of:
        padded = math.ceil(n / pad_to_multiple_of) * pad_to_multiple_of
        pad = padded - n
        if pad:
            q, k1, k2, v1, v2 = (torch.nn.functional.pad(t, (0, 0, 0, 0, 0, pad)) for t in (q, k1, k2, v1, v2))
    use_dense = dense if dense is not None else q.shape[1] <= 96
    fn = windowed_dense if use_dense else windowed_banded
    out, _ = fn(q, k1, k2, v1, v2, w1, w2)
    return out[:, :n]


# ---------------------------------------------------------------------------
# work counts used by the benchmark and its tests
# ---------------------------------------------------------------------------

def attended_triples(n: int, w1: int, w2: int) -> int:
    """Number of unmasked (i, j, k) triples per (batch, head)."""
    return sum(min(i + 1, w1) * min(i + 1, w2) for i in range(n))
