"""GPU parity of the multi-head module (triton_two_simplicial_attention.py:1062-1081 with
simplicial_mha.py:110-138 in the reference): the HIP-backed module against the same module
whose `attend` is the fp32 CPU oracle, sharing one state_dict."""
import pytest
import torch

from oracle import reference_attend as R

pytestmark = pytest.mark.gpu


def _pair(dim, heads, kv_heads, dim_head, w1, w2, seed, dim_head_values=None):
    from simplicial_attention_amd import SlidingWindowTwoSimplicialMHA
    from simplicial_attention_amd.simplicial_mha import HigherOrderAttention
    torch.manual_seed(seed)
    hip = SlidingWindowTwoSimplicialMHA(dim, dim_head=dim_head, heads=heads, key_value_heads=kv_heads, w1=w1, w2=w2,
                                        dim_head_values=dim_head_values)
    attend = lambda q, k, v: R.sliding_two_simplicial_attn(q, k, v, w1=w1, w2=w2)
    ref = HigherOrderAttention(dim, dim_head=dim_head, heads=heads, key_value_heads=kv_heads, attend=attend,
                               head_first_dim=False, dim_head_values=dim_head_values)
    ref.load_state_dict(hip.state_dict())
    # the oracle module computes in fp32 on the bf16-rounded weights
    hip = hip.bfloat16()
    ref.load_state_dict({k: v.float() for k, v in hip.state_dict().items()})
    return hip.cuda(), ref


def test_module_forward_config2():
    """benchmark config 2: tokens (2, 1024, 512), dim_head 64, 8 heads, w1=512, w2=32, bf16, forward."""
    hip, ref = _pair(512, 8, 8, 64, 512, 32, seed=1)
    tokens = torch.randn(2, 1024, 512, generator=torch.Generator().manual_seed(1)).bfloat16()
    with torch.no_grad():
        got = hip(tokens.cuda()).float().cpu()
        want = ref(tokens.float())
    err = (got - want).abs()
    # bf16 projections and norms around the kernel: the reference's own module test tolerance (atol 3e-2)
    assert float(err.max()) <= 3e-2, float(err.max())
    assert float(err.norm() / want.norm()) <= 2e-2


def test_module_forward_backward_grouped_heads():
    """Smaller module with grouped key/value heads (2 query heads per kv head): output and
    the gradients of tokens and of every parameter."""
    hip, ref = _pair(128, 4, 2, 64, 96, 16, seed=3)
    g = torch.Generator().manual_seed(4)
    tokens = torch.randn(2, 200, 128, generator=g).bfloat16()
    dout = torch.randn(2, 200, 128, generator=g).bfloat16()
    x_hip = tokens.cuda().requires_grad_(True)
    out = hip(x_hip)
    out.backward(dout.cuda())
    x_ref = tokens.float().requires_grad_(True)
    want = ref(x_ref)
    want.backward(dout.float())
    torch.cuda.synchronize()

    def rel(a, b):
        return float((a.float().cpu() - b).norm() / b.norm().clamp_min(1e-30))

    assert rel(out.detach(), want.detach()) <= 2e-2
    assert rel(x_hip.grad, x_ref.grad) <= 3e-2
    ref_params = dict(ref.named_parameters())
    for name, prm in hip.named_parameters():
        assert prm.grad is not None, name
        assert rel(prm.grad, ref_params[name].grad) <= 3e-2, (name, rel(prm.grad, ref_params[name].grad))


def test_module_with_narrow_value_heads_and_small_query_heads():
    """dim_head 32 with dim_head_values 16 (simplicial_mha.py:34,56 in the reference): the
    module takes the unfused norm path and the wrapper pads both to the kernels' 64."""
    hip, ref = _pair(128, 4, 2, 32, 64, 8, seed=5, dim_head_values=16)
    g = torch.Generator().manual_seed(6)
    tokens = torch.randn(2, 150, 128, generator=g).bfloat16()
    dout = torch.randn(2, 150, 128, generator=g).bfloat16()
    x_hip = tokens.cuda().requires_grad_(True)
    out = hip(x_hip)
    out.backward(dout.cuda())
    x_ref = tokens.float().requires_grad_(True)
    want = ref(x_ref)
    want.backward(dout.float())
    torch.cuda.synchronize()
    rel = lambda a, b: float((a.float().cpu() - b).norm() / b.norm().clamp_min(1e-30))
    assert rel(out.detach(), want.detach()) <= 2e-2
    assert rel(x_hip.grad, x_ref.grad) <= 3e-2


@pytest.mark.parametrize('heads,kv_heads,dim_head,n', [(8, 8, 64, 1024), (4, 2, 128, 333), (4, 4, 32, 257), (2, 1, 256, 130)])
def test_fused_qkv_norm_against_fp32_restatement(heads, kv_heads, dim_head, n):
    """The fused split + per-head RMSNorm kernel (simplicial_mha.py:116-127 in the reference)
    against the same arithmetic written with torch in fp32 on the bf16-rounded inputs:
    outputs within one bf16 rounding, gradients of the projection row and of the five
    weights through autograd of the restatement."""
    from simplicial_attention_amd.qkv_norm import FusedQKVNorm
    g = torch.Generator().manual_seed(7)
    b, eps = 2, 0.0078125
    channels = (heads + 4 * kv_heads) * dim_head
    qkv = torch.randn(b, n, channels, generator=g).bfloat16()
    ws = [(1 + 0.3 * torch.randn(dim_head, generator=g)).bfloat16() for _ in range(5)]
    douts = [torch.randn(b, n, h, dim_head, generator=g).bfloat16() for h in (heads, kv_heads, kv_heads, kv_heads, kv_heads)]

    x = qkv.cuda().requires_grad_(True)
    wd = [w.cuda().requires_grad_(True) for w in ws]
    outs = FusedQKVNorm.apply(x, *wd, heads, kv_heads, dim_head, eps)
    torch.autograd.backward(outs, [d.cuda() for d in douts])
    torch.cuda.synchronize()

    xr = qkv.float().requires_grad_(True)
    wr = [w.float().requires_grad_(True) for w in ws]
    qs, ks, vs = xr.split((heads * dim_head, 2 * kv_heads * dim_head, 2 * kv_heads * dim_head), dim=-1)
    rms = lambda t, w: t * torch.rsqrt(t.pow(2).mean(-1, keepdim=True) + eps) * w
    k1, k2 = ks.unflatten(-1, (kv_heads, 2 * dim_head)).chunk(2, dim=-1)
    v1, v2 = vs.unflatten(-1, (kv_heads, 2 * dim_head)).chunk(2, dim=-1)
    refs = [rms(qs.unflatten(-1, (heads, dim_head)), wr[0]), rms(k1, wr[1]), rms(k2, wr[2]), rms(v1, wr[3]), rms(v2, wr[4])]
    torch.autograd.backward(refs, [d.float() for d in douts])

    for got, ref in zip(outs, refs):
        assert got.shape == ref.shape and got.is_contiguous()
        assert torch.allclose(got.float().cpu(), ref.detach(), atol=1e-6, rtol=2 ** -8)      # one bf16 rounding
    assert torch.allclose(x.grad.float().cpu(), xr.grad, atol=2e-3, rtol=2 ** -7)
    for got, ref in zip(wd, wr):
        rel = float((got.grad.float().cpu() - ref.grad).norm() / ref.grad.norm())
        assert rel <= 5e-3, rel


def test_module_with_and_without_fused_norm_agree():
    from simplicial_attention_amd import SlidingWindowTwoSimplicialMHA
    torch.manual_seed(5)
    m = SlidingWindowTwoSimplicialMHA(256, dim_head=64, heads=4, key_value_heads=2, w1=64, w2=8).bfloat16().cuda()
    x = torch.randn(2, 150, 256, device='cuda').bfloat16()
    dout = torch.randn(2, 150, 256, device='cuda').bfloat16()

    def run(fused):
        m.fused_qkv_norm = fused
        m.zero_grad()
        xi = x.clone().requires_grad_(True)
        out = m(xi)
        out.backward(dout)
        return out.detach().float(), xi.grad.float(), {k: v.grad.float() for k, v in m.named_parameters()}

    out_f, dx_f, dp_f = run(True)
    out_u, dx_u, dp_u = run(False)
    rel = lambda a, b: float((a - b).norm() / b.norm().clamp_min(1e-30))
    assert rel(out_f, out_u) <= 1e-2 and rel(dx_f, dx_u) <= 2e-2
    for k in dp_u:
        assert rel(dp_f[k], dp_u[k]) <= 2e-2, (k, rel(dp_f[k], dp_u[k]))
