"""GPU parity of the multi-head module (triton_two_simplicial_attention.py:1062-1081 with
simplicial_mha.py:110-138 in the reference): the HIP-backed module against the same module
whose `attend` is the fp32 CPU oracle, sharing one state_dict."""
import pytest
import torch

from oracle import reference_attend as R

pytestmark = pytest.mark.gpu


def _pair(dim, heads, kv_heads, dim_head, w1, w2, seed):
    from simplicial_attention_amd import SlidingWindowTwoSimplicialMHA
    from simplicial_attention_amd.simplicial_mha import HigherOrderAttention
    torch.manual_seed(seed)
    hip = SlidingWindowTwoSimplicialMHA(dim, dim_head=dim_head, heads=heads, key_value_heads=kv_heads, w1=w1, w2=w2)
    attend = lambda q, k, v: R.sliding_two_simplicial_attn(q, k, v, w1=w1, w2=w2)
    ref = HigherOrderAttention(dim, dim_head=dim_head, heads=heads, key_value_heads=kv_heads, attend=attend,
                               head_first_dim=False)
    ref.load_state_dict(hip.state_dict())
    # the oracle module computes in fp32 on the bf16-rounded weights
    hip = hip.bfloat16()
    ref.load_state_dict({k: v.float() for k, v in hip.state_dict().items()})
    return hip.cuda(), ref


def test_module_forward_config2():
    """BASELINE config 2: tokens (2, 1024, 512), dim_head 64, 8 heads, w1=512, w2=32, bf16, forward."""
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
