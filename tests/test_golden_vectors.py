"""Frozen vectors (tests/golden/windowed_n20_d32_w9_w4.npz, written by tests/golden/make_vectors.py): the output and
lse of one small grouped-head case from Python loops over single (i, j, k) triples, its five gradients from central
differences of those loops.  Nothing in that arithmetic is shared with the oracle's tensor code, so a dropped term, a
wrong sign, an off-by-one window edge or a transposed operand in any oracle function fails here.  The GPU test puts the
HIP path against the same file."""
import os

import numpy as np
import pytest
import torch

from oracle import reference_attend as R
from oracle import c_oracle as C
from tests import parity_util as U

PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), 'golden', 'windowed_n20_d32_w9_w4.npz')
GRADS = ('dq', 'dk1', 'dk2', 'dv1', 'dv2')


def load():
    z = np.load(PATH)          # (plain arrays: allow_pickle stays off)
    shape = tuple(int(x) for x in z['shape'])
    t = lambda name: torch.from_numpy(z[name]).unsqueeze(0)
    ins = [t(name) for name in ('q', 'k1', 'k2', 'v1', 'v2', 'dout')]
    want = {name: t(name) for name in ('out',) + GRADS}
    want['lse'] = torch.from_numpy(z['lse']).unsqueeze(0)
    return shape, ins, want


def group_sum(t, hk, g):
    return t.unflatten(2, (hk, g)).sum(3)


def check(out, lse, grads, want, atol_fwd=1e-10, atol_grad=2e-8):
    assert torch.allclose(out.double(), want['out'], atol=atol_fwd, rtol=0)
    assert torch.allclose(lse.double(), want['lse'], atol=atol_fwd, rtol=0)
    for name, got in zip(GRADS, grads):
        assert torch.allclose(got.double(), want[name], atol=atol_grad, rtol=0), name


def test_banded_oracle_reproduces_the_vectors():
    (b, n, hq, hk, d, w1, w2), (q, k1, k2, v1, v2, dout), want = load()
    g = hq // hk
    ke = [R.expand_kv_heads(t, g) for t in (k1, k2, v1, v2)]
    out, lse, grads = R.windowed_banded_fwd_bwd(q, *ke, dout, w1, w2, chunk=7)
    check(out, lse, (grads[0], *(group_sum(t, hk, g) for t in grads[1:])), want)


def test_dense_oracle_and_explicit_gradients_reproduce_the_vectors():
    (b, n, hq, hk, d, w1, w2), (q, k1, k2, v1, v2, dout), want = load()
    g = hq // hk
    ke = [R.expand_kv_heads(t, g) for t in (k1, k2, v1, v2)]
    leaves = [t.clone().requires_grad_(True) for t in (q, *ke)]
    out, lse = R.windowed_dense(*leaves, w1, w2)
    auto = torch.autograd.grad(out, leaves, dout)
    check(out.detach(), lse.detach(), (auto[0], *(group_sum(t, hk, g) for t in auto[1:])), want)
    out_e, lse_e, delta, expl = R.windowed_grads_explicit(q, *ke, dout, w1, w2)
    check(out_e, lse_e, (expl[0], *(group_sum(t, hk, g) for t in expl[1:])), want)
    assert torch.allclose(delta, (want['out'] * dout).sum(-1).transpose(1, 2), atol=1e-10, rtol=0)


def test_c_oracle_reproduces_the_vectors():
    (b, n, hq, hk, d, w1, w2), (q, k1, k2, v1, v2, dout), want = load()
    g = hq // hk
    ke = [R.expand_kv_heads(t, g) for t in (k1, k2, v1, v2)]
    out, lse, grads = C.fwd_bwd(q, *ke, dout, w1, w2)
    check(out, lse, (grads[0], *(group_sum(t, hk, g) for t in grads[1:])), want)


def test_functional_wrapper_of_the_oracle_reproduces_the_vectors():
    """the oracle's restatement of the reference's wrapper (repeat of grouped heads, padding): output only"""
    (b, n, hq, hk, d, w1, w2), (q, k1, k2, v1, v2, dout), want = load()
    out = R.sliding_two_simplicial_attn(q, (k1, k2), (v1, v2), w1=w1, w2=w2, causal=True)
    assert torch.allclose(out.double(), want['out'], atol=1e-10, rtol=0)


@pytest.mark.gpu
def test_hip_path_reproduces_the_vectors():
    """bf16 kernels against the double-precision vectors: unit-variance inputs, so the reference's tolerances for such
    inputs apply beside the elementwise criterion (tests/parity_util.py)."""
    (b, n, hq, hk, d, w1, w2), ins, want = load()
    out, grads = U.hip_fwd_bwd(*(t.bfloat16() for t in ins), w1, w2)
    U.check_all(out, grads, want['out'], [want[name] for name in GRADS], unit_variance=True)
