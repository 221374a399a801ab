"""Pins for the CPU oracle (oracle/reference_attend.py, oracle/sa2_oracle.c).

The reference stores no golden vectors for this path, so each oracle function is
pinned by what the mathematics fixes: brute-force loops, a library routine
(scaled_dot_product_attention over the flattened N^2 key set, which is the
construction of the reference's tests/test_triton.py:52-64), closed-form special
cases, invariants and gradcheck.  Nothing here re-types the oracle's own formula.
"""
import itertools
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import reference_attend as R
from oracle import c_oracle as C

torch.set_default_dtype(torch.float32)


def rand(*shape, seed=0, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g, dtype=dtype)


def five(b, n, h, d, seed=0, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    return [torch.randn(b, n, h, d, generator=g, dtype=dtype) for _ in range(5)]


def brute_force(q, k1, k2, v1, v2, w1, w2):
    """Python loops over single numbers, one (i, j, k) at a time."""
    b, n, h, d = q.shape
    out = torch.zeros_like(q)
    lse = torch.zeros(b, h, n, dtype=q.dtype)
    scale = d ** -0.5
    for bi, hi, i in itertools.product(range(b), range(h), range(n)):
        logits, vals = [], []
        for j in range(n):
            for k in range(n):
                if not (0 <= i - j < w1 and 0 <= i - k < w2):
                    continue
                s = sum(float(q[bi, i, hi, c]) * float(k1[bi, j, hi, c]) * float(k2[bi, k, hi, c]) for c in range(d))
                logits.append(s * scale)
                vals.append([float(v1[bi, j, hi, c]) * float(v2[bi, k, hi, c]) for c in range(d)])
        m = max(logits)
        z = sum(math.exp(s - m) for s in logits)
        lse[bi, hi, i] = m + math.log(z)
        for c in range(d):
            out[bi, i, hi, c] = sum(math.exp(s - m) / z * v[c] for s, v in zip(logits, vals))
    return out, lse


@pytest.mark.parametrize('w1,w2', [(1, 1), (2, 3), (3, 2), (8, 8), (4, 1), (1, 4)])
def test_dense_matches_brute_force(w1, w2):
    q, k1, k2, v1, v2 = five(1, 7, 2, 3, seed=w1 * 10 + w2)
    out, lse = R.windowed_dense(q, k1, k2, v1, v2, w1, w2)
    bo, bl = brute_force(q, k1, k2, v1, v2, w1, w2)
    assert torch.allclose(out, bo, atol=1e-12)
    assert torch.allclose(lse, bl, atol=1e-12)


@pytest.mark.parametrize('w1,w2', [(5, 3), (16, 4), (40, 40)])
def test_dense_matches_sdpa_over_flattened_keys(w1, w2):
    """Library routine: softmax attention over N^2 keys k1_j*k2_k, values v1_j*v2_k,
    with the band mask (tests/test_triton.py:33-64 in the reference)."""
    b, n, h, d = 2, 24, 2, 16
    q, k1, k2, v1, v2 = five(b, n, h, d, seed=3)
    qh, a1, a2, b1, b2 = (t.permute(0, 2, 1, 3) for t in (q, k1, k2, v1, v2))
    kk = (a1[:, :, :, None, :] * a2[:, :, None, :, :]).reshape(b, h, n * n, d)
    vv = (b1[:, :, :, None, :] * b2[:, :, None, :, :]).reshape(b, h, n * n, d)
    idx = torch.arange(n)
    kv = torch.arange(n * n)
    d1 = idx[:, None] - (kv // n)[None, :]
    d2 = idx[:, None] - (kv % n)[None, :]
    mask = (d1 >= 0) & (d1 < w1) & (d2 >= 0) & (d2 < w2)
    ref = F.scaled_dot_product_attention(qh, kk, vv, attn_mask=mask).permute(0, 2, 1, 3)
    out, _ = R.windowed_dense(q, k1, k2, v1, v2, w1, w2)
    assert torch.allclose(out, ref, atol=1e-10)


def test_unit_second_set_reduces_to_sliding_window_attention():
    """k2 = v2 = 1 : per-row multiplicity of k cancels in the softmax, leaving plain
    causal sliding-window(w1) attention; symmetric statement for the first set."""
    b, n, h, d = 1, 33, 2, 8
    q, k1, k2, v1, v2 = five(b, n, h, d, seed=5)
    ones = torch.ones_like(k2)
    idx = torch.arange(n)
    for w1, w2 in [(6, 4), (33, 2), (3, 33)]:
        out, _ = R.windowed_dense(q, k1, ones, v1, ones, w1, w2)
        dlt = idx[:, None] - idx[None, :]
        ref = F.scaled_dot_product_attention(q.permute(0, 2, 1, 3), k1.permute(0, 2, 1, 3), v1.permute(0, 2, 1, 3),
                                             attn_mask=(dlt >= 0) & (dlt < w1)).permute(0, 2, 1, 3)
        assert torch.allclose(out, ref, atol=1e-10)
        out, _ = R.windowed_dense(q, ones, k2, ones, v2, w1, w2)
        ref = F.scaled_dot_product_attention(q.permute(0, 2, 1, 3), k2.permute(0, 2, 1, 3), v2.permute(0, 2, 1, 3),
                                             attn_mask=(dlt >= 0) & (dlt < w2)).permute(0, 2, 1, 3)
        assert torch.allclose(out, ref, atol=1e-10)


def test_unit_values_give_unit_output_and_lse_counts_triples():
    b, n, h, d = 1, 20, 1, 4
    q, k1, k2, v1, v2 = five(b, n, h, d, seed=6)
    out, _ = R.windowed_dense(q, k1, k2, torch.ones_like(v1), torch.ones_like(v2), 5, 3)
    assert torch.allclose(out, torch.ones_like(out), atol=1e-12)
    # zero queries: every logit is 0, so lse_i = log(#attended (j,k) pairs of row i)
    _, lse = R.windowed_dense(torch.zeros_like(q), k1, k2, v1, v2, 5, 3)
    want = torch.tensor([math.log(min(i + 1, 5) * min(i + 1, 3)) for i in range(n)], dtype=lse.dtype)
    assert torch.allclose(lse[0, 0], want, atol=1e-12)
    assert R.attended_triples(n, 5, 3) == round(float(torch.exp(lse[0, 0]).sum()))


def test_windows_at_least_n_equal_full_causal_naive():
    """w1, w2 >= N is the reference's dense causal operator
    (simplicial_attention.py:111-117), here in its own head-first layout with GQA."""
    b, n, hq, hk, d = 2, 12, 4, 2, 8
    g = torch.Generator().manual_seed(7)
    q = torch.randn(b, n, hq, d, generator=g, dtype=torch.float64)
    k1, k2, v1, v2 = [torch.randn(b, n, hk, d, generator=g, dtype=torch.float64) for _ in range(4)]
    ref = R.naive_two_simplicial_attend(q.permute(0, 2, 1, 3), (k1.permute(0, 2, 1, 3), k2.permute(0, 2, 1, 3)),
                                        (v1.permute(0, 2, 1, 3), v2.permute(0, 2, 1, 3)), causal=True).permute(0, 2, 1, 3)
    out = R.sliding_two_simplicial_attn(q, (k1, k2), (v1, v2), w1=n, w2=n + 5, pad_to_multiple_of=8)
    assert torch.allclose(out, ref, atol=1e-10)
    # GQA: query head h*g + r reads kv head h ('(h g)' order)
    for head in range(hq):
        solo = R.windowed_dense(q[:, :, head:head + 1], k1[:, :, head // 2:head // 2 + 1], k2[:, :, head // 2:head // 2 + 1],
                                v1[:, :, head // 2:head // 2 + 1], v2[:, :, head // 2:head // 2 + 1], n, n)[0]
        assert torch.allclose(out[:, :, head:head + 1], solo, atol=1e-10)


def test_naive_non_causal_matches_flat_softmax():
    b, h, n, d = 1, 2, 6, 4
    g = torch.Generator().manual_seed(8)
    q, k1, k2, v1, v2 = [torch.randn(b, h, n, d, generator=g, dtype=torch.float64) for _ in range(5)]
    kk = (k1[:, :, :, None] * k2[:, :, None]).reshape(b, h, n * n, d)
    vv = (v1[:, :, :, None] * v2[:, :, None]).reshape(b, h, n * n, d)
    ref = F.scaled_dot_product_attention(q, kk, vv)
    out = R.naive_two_simplicial_attend(q, (k1, k2), (v1, v2), causal=False)
    assert torch.allclose(out, ref, atol=1e-10)


def test_invariants_causality_locality_independence_symmetry():
    b, n, h, d = 2, 30, 2, 4
    w1, w2 = 7, 3
    q, k1, k2, v1, v2 = five(b, n, h, d, seed=9)
    base, _ = R.windowed_dense(q, k1, k2, v1, v2, w1, w2)
    # causality: changing rows > t leaves rows <= t untouched
    t = 17
    q2, k12, k22, v12, v22 = (x.clone() for x in (q, k1, k2, v1, v2))
    for x in (q2, k12, k22, v12, v22):
        x[:, t + 1:] += 3.0
    pert, _ = R.windowed_dense(q2, k12, k22, v12, v22, w1, w2)
    assert torch.equal(pert[:, :t + 1], base[:, :t + 1])
    # locality: row i ignores k1/v1 rows <= i-w1 and k2/v2 rows <= i-w2
    i = 20
    k13, v13, k23, v23 = (x.clone() for x in (k1, v1, k2, v2))
    k13[:, :i - w1 + 1] = 9.0
    v13[:, :i - w1 + 1] = -9.0
    k23[:, :i - w2 + 1] = 9.0
    v23[:, :i - w2 + 1] = -9.0
    loc, _ = R.windowed_dense(q, k13, k23, v13, v23, w1, w2)
    assert torch.allclose(loc[:, i], base[:, i], atol=1e-12)
    assert not torch.allclose(loc[:, i - 1], base[:, i - 1], atol=1e-3)
    # batch / head independence
    solo, _ = R.windowed_dense(q[1:, :, 1:], k1[1:, :, 1:], k2[1:, :, 1:], v1[1:, :, 1:], v2[1:, :, 1:], w1, w2)
    assert torch.allclose(solo, base[1:, :, 1:], atol=1e-12)
    # symmetry under swapping the two key/value sets together with their windows
    swapped, _ = R.windowed_dense(q, k2, k1, v2, v1, w2, w1)
    assert torch.allclose(swapped, base, atol=1e-12)


@pytest.mark.parametrize('n,w1,w2,chunk', [(50, 9, 4, 16), (50, 64, 3, 7), (33, 5, 40, 32), (64, 16, 8, 64)])
def test_banded_equals_dense(n, w1, w2, chunk):
    q, k1, k2, v1, v2 = five(2, n, 2, 8, seed=n + w1)
    do = rand(2, n, 2, 8, seed=99)
    od, ld = R.windowed_dense(q, k1, k2, v1, v2, w1, w2)
    ob, lb = R.windowed_banded(q, k1, k2, v1, v2, w1, w2, chunk=chunk)
    assert torch.allclose(od, ob, atol=1e-12) and torch.allclose(ld, lb, atol=1e-12)
    _, _, _, ge = R.windowed_grads_explicit(q, k1, k2, v1, v2, do, w1, w2)
    _, _, gb = R.windowed_banded_fwd_bwd(q, k1, k2, v1, v2, do, w1, w2, chunk=chunk)
    for a, bb in zip(ge, gb):
        assert torch.allclose(a, bb, atol=1e-11)


def test_explicit_gradients_match_autograd_and_gradcheck():
    b, n, h, d = 1, 9, 2, 3
    w1, w2 = 4, 2
    ts = [t.requires_grad_(True) for t in five(b, n, h, d, seed=11)]
    do = rand(b, n, h, d, seed=12)
    out, _ = R.windowed_dense(*ts, w1, w2)
    auto = torch.autograd.grad((out * do).sum(), ts)
    _, _, _, expl = R.windowed_grads_explicit(*[t.detach() for t in ts], do, w1, w2)
    for a, e in zip(auto, expl):
        assert torch.allclose(a, e, atol=1e-12)
    assert torch.autograd.gradcheck(lambda *x: R.windowed_dense(*x, w1, w2)[0], ts, eps=1e-6, atol=1e-6)


@pytest.mark.parametrize('w1,w2', [(7, 3), (24, 24), (1, 1), (5, 9)])
def test_c_restatement_matches_torch_restatement(w1, w2):
    q, k1, k2, v1, v2 = five(2, 24, 2, 8, seed=13)
    do = rand(2, 24, 2, 8, seed=14)
    co, cl, cg = C.fwd_bwd(q, k1, k2, v1, v2, do, w1, w2)
    to, tl, _, tg = R.windowed_grads_explicit(q, k1, k2, v1, v2, do, w1, w2)
    assert torch.allclose(co, to, atol=1e-12) and torch.allclose(cl, tl, atol=1e-12)
    for a, bb in zip(cg, tg):
        assert torch.allclose(a, bb, atol=1e-12)


def test_c_restatement_matches_brute_force():
    q, k1, k2, v1, v2 = five(1, 6, 1, 2, seed=15)
    co, cl, _ = C.fwd_bwd(q, k1, k2, v1, v2, None, 3, 2)
    bo, bl = brute_force(q, k1, k2, v1, v2, 3, 2)
    assert torch.allclose(co, bo, atol=1e-12) and torch.allclose(cl, bl, atol=1e-12)


def test_config1_shape_fp32_naive_and_grads():
    """benchmark config 1: B=1, H=4, N=128, D=32, fp32, causal; the dense naive
    restatement against the banded oracle with windows >= N, output and five grads."""
    g = torch.Generator().manual_seed(0)
    q, k1, k2, v1, v2, do = [torch.randn(1, 4, 128, 32, generator=g) for _ in range(6)]
    ts = [t.clone().requires_grad_(True) for t in (q, k1, k2, v1, v2)]
    out = R.naive_two_simplicial_attend(ts[0], (ts[1], ts[2]), (ts[3], ts[4]), causal=True)
    grads = torch.autograd.grad((out * do).sum(), ts)
    perm = lambda t: t.permute(0, 2, 1, 3).double()
    bo, _, bg = R.windowed_banded_fwd_bwd(*[perm(t) for t in (q, k1, k2, v1, v2)], perm(do), 128, 128, chunk=32)
    assert torch.allclose(perm(out), bo, atol=2e-5)
    for a, e in zip(grads, bg):
        assert torch.allclose(perm(a), e, atol=1e-4, rtol=1e-4)


def test_triple_count_formula():
    assert R.attended_triples(128, 128, 128) == sum((i + 1) ** 2 for i in range(128)) == 707264
    assert R.attended_triples(8192, 512, 32) == 130026160
    assert R.attended_triples(1024, 512, 32) == 12585648
    mask = R.window_mask(40, 9, 4)
    assert int(mask.sum()) == R.attended_triples(40, 9, 4)
