"""Parity at the full sizes of the benchmark configurations.

The CPU oracle cannot cover all (batch, head) slices of these shapes in test time, so:
  * one complete (batch, head) slice of config 3 is checked against the banded fp32 oracle
    (forward and all five gradients, all 8192 rows), and the other slices through batch /
    head independence: permuting the slices of the inputs permutes the outputs bit for bit;
  * the layer shape of config 5 (grouped heads, dim_head 64) the same way;
  * config 4 (N = 32768) is checked through translation equivariance of the windows: the
    last rows of the full sequence must equal a run on the cropped sequence that still
    holds every row those queries can reach.
"""
import pytest
import torch

from tests import parity_util as U

pytestmark = pytest.mark.gpu


def _run(q, k1, k2, v1, v2, dout, w1, w2):
    from simplicial_attention_amd import sliding_two_simplicial_attn
    ts = [t.detach().requires_grad_(True) for t in (q, k1, k2, v1, v2)]
    out = sliding_two_simplicial_attn(ts[0], (ts[1], ts[2]), (ts[3], ts[4]), w1=w1, w2=w2, causal=True)
    grads = torch.autograd.grad(out, ts, dout)
    torch.cuda.synchronize()
    return out.detach(), grads


def test_config3_one_slice_against_oracle_and_slice_independence():
    b, n, h, d, w1, w2 = 4, 8192, 8, 128, 512, 32
    g = torch.Generator(device='cpu').manual_seed(2)
    mk = lambda s: (torch.randn(b, n, h, d, generator=g) * s).bfloat16()
    q, k1, k2, v1, v2 = (mk(d ** -0.5) for _ in range(5))
    dout = mk(1.0)
    dev = [t.cuda() for t in (q, k1, k2, v1, v2, dout)]
    out, grads = _run(*dev, w1, w2)

    # one slice, every row, forward and backward, against the CPU oracle
    sb, sh = 3, 5
    cut = lambda t: t[sb:sb + 1, :, sh:sh + 1].contiguous()
    ref_out, _, ref_grads = U.oracle_fwd_bwd(*(cut(t) for t in (q, k1, k2, v1, v2, dout)), w1, w2)
    U.check_all(cut(out.cpu()), [cut(t.cpu()) for t in grads], ref_out, ref_grads)

    # the other slices: reversing batch and head order of the inputs reverses the outputs exactly
    flip = lambda t: t.flip(0).flip(2).contiguous()
    out_f, grads_f = _run(*(flip(t) for t in dev), w1, w2)
    assert torch.equal(flip(out_f), out)
    for a, b_ in zip(grads_f, grads):
        assert torch.equal(flip(a), b_)


def test_config5_layer_one_group_against_oracle_and_slice_independence():
    """Shape of one simplicial layer of config 5: B=8, N=2048, 8 query heads on 4 key/value
    heads, dim_head 64 (at this head size dK1 and dV1 come from one kernel).  One batch entry
    and one key/value head with its two query heads against the oracle, the rest through
    batch / head independence."""
    b, n, hq, hk, d, w1, w2 = 8, 2048, 8, 4, 64, 512, 32
    ins = U.make_inputs(b, n, hq, hk, d, seed=4, std=d ** -0.5)
    dev = [t.cuda() for t in ins]
    out, grads = _run(*dev, w1, w2)
    sb, sk = 5, 2
    cut_q = lambda t: t[sb:sb + 1, :, 2 * sk:2 * sk + 2].contiguous()
    cut_k = lambda t: t[sb:sb + 1, :, sk:sk + 1].contiguous()
    q, k1, k2, v1, v2, dout = ins
    ref_out, _, ref_grads = U.oracle_fwd_bwd(cut_q(q), cut_k(k1), cut_k(k2), cut_k(v1), cut_k(v2), cut_q(dout), w1, w2)
    U.check_all(cut_q(out.cpu()), [cut_q(grads[0].cpu())] + [cut_k(t.cpu()) for t in grads[1:]], ref_out, ref_grads)
    # reversing the batch order and the order of the key/value heads (query heads move with their group)
    flip_k = lambda t: t.flip(0).flip(2).contiguous()
    flip_q = lambda t: t.flip(0).unflatten(2, (hk, hq // hk)).flip(2).flatten(2, 3).contiguous()
    flips = (flip_q, flip_k, flip_k, flip_k, flip_k, flip_q)
    out_f, grads_f = _run(*(f(t) for f, t in zip(flips, dev)), w1, w2)
    assert torch.equal(flip_q(out_f), out)
    for f, a, b_ in zip(flips[:5], grads_f, grads):
        assert torch.equal(f(a), b_)


def test_config4_translation_equivariance():
    b, n, h, d, w1, w2 = 1, 32768, 16, 128, 512, 32
    g = torch.Generator(device='cpu').manual_seed(3)
    mk = lambda s: (torch.randn(b, n, h, d, generator=g) * s).bfloat16().cuda()
    q, k1, k2, v1, v2 = (mk(d ** -0.5) for _ in range(5))
    dout = mk(1.0)
    out, grads = _run(q, k1, k2, v1, v2, dout, w1, w2)
    # rows >= first can only see rows >= first - (w1 - 1); crop at a tile-unaligned position
    first, start = 30011, 30011 - (w1 - 1)
    crop = lambda t: t[:, start:].contiguous()
    out_c, grads_c = _run(*(crop(t) for t in (q, k1, k2, v1, v2, dout)), w1, w2)
    off = first - start
    # the cropped run tiles the sequence differently, so sums are ordered differently:
    # equality up to bf16 rounding of the outputs
    close = lambda a, b_: torch.allclose(a.float(), b_.float(), atol=2e-2, rtol=1e-2)
    assert close(out[:, first:], out_c[:, off:])
    assert close(grads[0][:, first:], grads_c[0][:, off:])                    # dq: a row's gradient needs its own window only
    for a, c_ in zip(grads[1:], grads_c[1:]):                                 # dk1, dk2, dv1, dv2: rows fed only by queries >= first
        assert close(a[:, first:], c_[:, off:])
    rel = lambda a, b_: float((a.float() - b_.float()).norm() / b_.float().norm())
    assert rel(out[:, first:], out_c[:, off:]) <= 1e-2
    for a, c_ in zip(grads, grads_c):
        assert rel(a[:, first:], c_[:, off:]) <= 1e-2
