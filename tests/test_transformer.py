"""The decoder stack and LM wrapper (two_simplicial_transformer.py:24-141 and train.py:64-135
of the reference): structure on the CPU, parity of a small model on the GPU against the same
model whose simplicial layers call the fp32 CPU oracle."""
from functools import partial

import pytest
import torch

from oracle import reference_attend as R
from simplicial_attention_amd.two_simplicial_attention import SlidingWindowTwoSimplicialMHA
from simplicial_attention_amd.two_simplicial_transformer import Attention, TwoSimplicialLM, TwoSimplicialTransformer


def test_layer_placement_and_parameter_names():
    m = TwoSimplicialTransformer(128, depth=8, heads=4, key_value_heads=2, dim_head=64, two_simplicial_attn_every=4)
    kinds = [type(attn) for attn, _ in m.layers]
    assert [k is SlidingWindowTwoSimplicialMHA for k in kinds] == [False, False, False, True] * 2
    assert all(k in (Attention, SlidingWindowTwoSimplicialMHA) for k in kinds)
    keys = set(m.state_dict())
    # names of the reference's modules: ordinary layer, simplicial layer (prenorm=True), feed-forward, final norm
    for k in ('layers.0.0.prenorm.weight', 'layers.0.0.to_q.weight', 'layers.0.0.to_kv.weight', 'layers.0.0.to_out.weight',
              'layers.3.0.prenorm.weight', 'layers.3.0.to_qkv.weight', 'layers.3.0.q_norm.weight',
              'layers.3.0.k_norms.1.weight', 'layers.3.0.v_norms.0.weight', 'layers.3.0.combine_heads.weight',
              'layers.0.1.0.weight', 'layers.0.1.1.weight', 'layers.0.1.1.bias', 'layers.0.1.3.weight', 'norm.weight'):
        assert k in keys, k
    assert m.state_dict()['layers.0.0.to_kv.weight'].shape == (2 * 2 * 64, 128)
    assert m.state_dict()['layers.3.0.to_qkv.weight'].shape == (4 * 64 + 2 * 2 * 2 * 64, 128)


def test_ordinary_attention_layer_is_grouped_causal_softmax_attention():
    torch.manual_seed(0)
    a = Attention(32, dim_head=8, heads=4, key_value_heads=2)
    x = torch.randn(2, 10, 32)
    got = a(x)
    xn = torch.nn.functional.rms_norm(x, (32,), a.prenorm.weight)
    q = (xn @ a.to_q.weight.t()).view(2, 10, 4, 8)
    kv = (xn @ a.to_kv.weight.t()).view(2, 10, 2, 2, 8)
    out = torch.zeros(2, 10, 4, 8)
    for h in range(4):
        k, v = kv[:, :, 0, h // 2], kv[:, :, 1, h // 2]
        s = torch.einsum('bid,bjd->bij', q[:, :, h], k) * 8 ** -0.5
        s = s.masked_fill(torch.ones(10, 10).triu(1).bool(), float('-inf'))
        out[:, :, h] = torch.einsum('bij,bjd->bid', s.softmax(-1), v)
    want = out.reshape(2, 10, 32) @ a.to_out.weight.t()
    assert torch.allclose(got, want, atol=1e-5)


@pytest.mark.gpu
def test_small_language_model_loss_and_gradients_on_gpu():
    torch.manual_seed(3)
    kw = dict(num_tokens=256, dim=128, depth=4, max_seq_len=160, dim_head=64, heads=4, two_simplicial_attn_every=2,
              transformer_kwargs=dict(key_value_heads=2, two_simplicial_attn_kwargs=dict(w1=48, w2=8, qk_rmsnorm=True)))
    hip = TwoSimplicialLM(**kw).bfloat16()
    ref = TwoSimplicialLM(**kw)
    ref.load_state_dict({k: v.float() for k, v in hip.state_dict().items()})
    for attn, _ in ref.transformer.layers:
        if isinstance(attn, SlidingWindowTwoSimplicialMHA):
            attn.attend = partial(R.sliding_two_simplicial_attn, w1=48, w2=8)
    tokens = torch.randint(0, 256, (2, 161), generator=torch.Generator().manual_seed(5))
    hip = hip.cuda()
    loss = hip(tokens.cuda(), return_loss=True)
    loss.backward()
    want = ref(tokens, return_loss=True)
    want.backward()
    torch.cuda.synchronize()
    assert abs(loss.item() - want.item()) <= 2e-2 * abs(want.item()), (loss.item(), want.item())
    ref_grads = dict(ref.named_parameters())
    worst = 0.0
    for name, prm in hip.named_parameters():
        g, r = prm.grad.float().cpu(), ref_grads[name].grad
        rel = float((g - r).norm() / r.norm().clamp_min(1e-30))
        worst = max(worst, rel)
        assert rel <= 4e-2, (name, rel)      # bf16 parameters, activations and 4 layers of bf16 matmuls against an fp32 model
    print('largest relative gradient error', worst)
