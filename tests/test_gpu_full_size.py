"""Parity at the full sizes of the benchmark configurations.

The CPU oracle cannot cover all (batch, head) slices of these shapes in test time, so:
  * one complete (batch, head) slice of config 3 is checked against the banded fp32 oracle
    (forward and all five gradients, all 8192 rows), and the other slices through batch /
    head independence: permuting the slices of the inputs permutes the outputs bit for bit;
  * the layer shape of config 5 (grouped heads, dim_head 64) the same way;
  * config 4 (N = 32768): one complete (batch, head) slice against the banded fp32 oracle
    (all 32768 rows, forward and five gradients), and translation equivariance of the
    windows: the last rows of the full sequence must equal a run on the cropped sequence
    that still holds every row those queries can reach;
  * config 1 exactly (the reference's CPU-runnable case: B=1, H=4, N=128, D=32, float32
    N(0,1) inputs, full causal): the HIP path with both windows = N against autograd
    through the dense naive attend.
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


def test_config4_one_slice_against_oracle():
    """One complete (batch, head) slice of config 4, all 32768 rows: output and the five
    gradients against the banded fp32 CPU oracle (about 15 s of CPU time)."""
    b, n, h, d, w1, w2 = 1, 32768, 16, 128, 512, 32
    g = torch.Generator(device='cpu').manual_seed(3)
    mk = lambda s: (torch.randn(b, n, h, d, generator=g) * s).bfloat16()
    q, k1, k2, v1, v2 = (mk(d ** -0.5) for _ in range(5))
    dout = mk(1.0)
    out, grads = _run(*(t.cuda() for t in (q, k1, k2, v1, v2, dout)), w1, w2)
    sh = 11
    cut = lambda t: t[:, :, sh:sh + 1].contiguous()
    ref_out, _, ref_grads = U.oracle_fwd_bwd(*(cut(t) for t in (q, k1, k2, v1, v2, dout)), w1, w2)
    U.check_all(cut(out.cpu()), [cut(t.cpu()) for t in grads], ref_out, ref_grads)


def test_config1_full_causal_against_dense_naive_attend():
    """benchmark config 1 on the HIP path: B=1, H=4, N=128, D=32, float32 N(0,1) inputs from a
    fixed seed, full causal (both windows = N, the case of the reference's test_triton.py:65-80),
    output and the autograd gradients of all five inputs against the dense naive attend
    (simplicial_attention.py:78-127 restated in oracle/reference_attend.py, layout b h n d).
    The kernels compute on bf16 operands: the oracle takes the bf16-rounded values, and the
    reference's own tolerances for unit-variance inputs apply (tests/parity_util.py)."""
    from oracle import reference_attend as R
    from simplicial_attention_amd import sliding_two_simplicial_attn
    b, h, n, d = 1, 4, 128, 32
    g = torch.Generator(device='cpu').manual_seed(0)
    q, k1, k2, v1, v2, dout = (torch.randn(b, h, n, d, generator=g) for _ in range(6))      # b h n d, float32
    rounded = [t.bfloat16().float() for t in (q, k1, k2, v1, v2, dout)]
    leaves = [t.clone().requires_grad_(True) for t in rounded[:5]]
    ref_out = R.naive_two_simplicial_attend(leaves[0], (leaves[1], leaves[2]), (leaves[3], leaves[4]), causal=True)
    ref_grads = torch.autograd.grad(ref_out, leaves, rounded[5])
    to_kernel = lambda t: t.transpose(1, 2).contiguous()                                    # b n h d
    ts = [to_kernel(t).cuda().requires_grad_(True) for t in (q, k1, k2, v1, v2)]
    out = sliding_two_simplicial_attn(ts[0], (ts[1], ts[2]), (ts[3], ts[4]), w1=n, w2=n, causal=True)
    assert out.dtype is torch.float32 and out.shape == (b, n, h, d)
    grads = torch.autograd.grad(out, ts, to_kernel(dout).cuda())
    U.check_all(out, grads, to_kernel(ref_out.detach()), [to_kernel(t) for t in ref_grads], unit_variance=True)


@pytest.mark.parametrize('n, seed', [(8192, 12), (32768, 13)])
def test_full_length_slices_with_unit_variance_inputs(n, seed):
    """One (batch, head) slice at the sequence lengths of configs 3 and 4 (D = 128, w1 = 512, w2 = 32) with
    UNSCALED N(0,1) inputs: the benchmark distribution N(0,1)/sqrt(D) makes outputs of order 1e-4, where only
    the relative bound binds; here logits have unit variance and outputs are of order one, so the elementwise
    criterion binds on every row of the full sequence.  Against the banded fp32 oracle, with the reference's own
    tolerances for such inputs (tests/test_triton.py:104-115) plus the relative Frobenius bound."""
    d, w1, w2 = 128, 512, 32
    ins = U.make_inputs(1, n, 1, 1, d, seed=seed, std=1.0)
    ref_out, _, ref_grads = U.oracle_fwd_bwd(*ins, w1, w2)
    out, grads = _run(*(t.cuda() for t in ins), w1, w2)
    U.check_all(out.cpu(), [t.cpu() for t in grads], ref_out, ref_grads, unit_variance=True)


@pytest.mark.parametrize('std', [None, 1.0], ids=['std_rsqrt_d', 'std_1'])
def test_head_dimension_256_long_slice_against_oracle(std):
    """Head dimension 256 at a length where every query tile walks the full first window many times over: one
    (batch, key/value head) group of two query heads, N = 2048, default windows, against the banded fp32 oracle.
    At the benchmark's input scale every element meets |x - ref| <= 2e-2 + 1e-2 |ref|.  With unscaled N(0,1) inputs
    the bf16 rounding of q * k2 and do * v2 enters a contraction twice as long as at D = 128 and one gradient element
    in 10^6 lands at 2.6e-2 where the criterion allows 2.3e-2: that run is judged by the reference's own tolerances
    for such inputs (3e-2 / 5e-2 absolute, tests/test_triton.py:104-115) plus the relative Frobenius bound of 1e-2."""
    n, d, w1, w2 = 2048, 256, 512, 32
    ins = U.make_inputs(1, n, 2, 1, d, seed=17, std=d ** -0.5 if std is None else std)
    ref_out, _, ref_grads = U.oracle_fwd_bwd(*ins, w1, w2)
    out, grads = _run(*(t.cuda() for t in ins), w1, w2)
    U.check_all(out.cpu(), [t.cpu() for t in grads], ref_out, ref_grads, unit_variance=std is not None, reference_atol_only=std is not None)


def test_config5_full_training_step_is_finite_and_deterministic():
    """benchmark config 5 at full size: the byte-level language model (depth 12, dim 512, 8 heads of 64 on 4
    key/value heads, every 2nd layer simplicial with w1 = 512, w2 = 32) on a batch of 8 x 2048 random bytes, bf16.
    One forward + backward: the loss of the untrained model is close to ln 256, every gradient is finite, and a
    second run gives the same loss and the same gradients bit for bit (no atomics anywhere on the path)."""
    import math
    from simplicial_attention_amd.two_simplicial_transformer import TwoSimplicialLM
    torch.manual_seed(4)
    lm = TwoSimplicialLM(num_tokens=256, dim=512, depth=12, max_seq_len=2048, dim_head=64, heads=8,
                         two_simplicial_attn_every=2, transformer_kwargs=dict(key_value_heads=4)).bfloat16().cuda()
    tokens = torch.randint(0, 256, (8, 2049), generator=torch.Generator().manual_seed(6)).cuda()

    def run():
        lm.zero_grad(set_to_none=True)
        loss = lm(tokens, return_loss=True)
        loss.backward()
        torch.cuda.synchronize()
        return loss.item(), {k: p.grad.clone() for k, p in lm.named_parameters()}
    loss_a, grads_a = run()
    loss_b, grads_b = run()
    print('   loss', loss_a, 'ln 256 =', math.log(256), flush=True)
    assert math.isfinite(loss_a) and abs(loss_a - math.log(256)) <= 0.5, loss_a
    assert loss_a == loss_b
    for name, g in grads_a.items():
        assert torch.isfinite(g).all(), name
        assert float(g.float().norm()) > 0, name
    # the simplicial layers' own parameters must be reproduced bit for bit (the library has no atomics); the other
    # layers go through torch's kernels, which are deterministic for these shapes too
    for name, g in grads_a.items():
        assert torch.equal(g, grads_b[name]), name
