"""CPU-side checks: the C-ABI library loads, exports every symbol that include/sa2.h
declares, validates its arguments before touching a device; the Python front end
keeps the reference's names, defaults, parameter names and error behaviour."""
import ctypes
import os
import re

import pytest
import torch

from simplicial_attention_amd import _native
import simplicial_attention_amd as S
from oracle import reference_attend as R

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope='module')
def lib():
    if not os.path.exists(_native.LIB_PATH):
        _native.build()
    return _native.load()


def header_symbols():
    text = open(os.path.join(ROOT, 'include', 'sa2.h')).read()
    text = re.sub(r'/\*.*?\*/', '', text, flags=re.S)
    return sorted(set(re.findall(r'\b(sa2_[a-z0-9_]+)\s*\(', text)))


def test_every_declared_symbol_is_exported(lib):
    names = header_symbols()
    assert set(names) == set(_native.EXPORTS)
    for name in names:
        assert getattr(lib, name) is not None
    assert lib.sa2_version() == 102


def test_supported_matrix(lib):
    assert lib.sa2_supported(64, 512, 32, 0) == 1
    assert lib.sa2_supported(128, 512, 64, 0) == 1
    assert lib.sa2_supported(128, 512, 65, 0) == 1
    assert lib.sa2_supported(64, 8192, 8192, 0) == 1
    assert lib.sa2_supported(32, 512, 32, 0) == 1
    assert lib.sa2_supported(96, 512, 32, 0) == 0
    assert lib.sa2_supported(256, 512, 32, 0) == 1
    assert lib.sa2_supported(512, 512, 32, 0) == 0
    assert lib.sa2_supported(128, 0, 32, 0) == 0
    assert lib.sa2_supported(128, 512, 32, 1) == 0


def _dummy(ptr=0x1000, sb=1024, sn=128, sh=8):
    return _native.TensorArg(ptr, sb, sn, sh)


def test_head_dimension_256_keeps_no_forward_partials(lib):
    """The kernels of head dimension 256 recompute in the backward: the size queries say 0 and a call that passes
    saved partials anyway is refused before any launch."""
    prob = _native.problem(1, 64, 2, 1, 256, 512, 32, True, 256 ** -0.5)
    assert lib.sa2_saved_t_bytes(prob) == 0 and lib.sa2_saved_m_bytes(prob) == 0
    assert lib.sa2_bwd_workspace_bytes(prob) == 2 * 1 * 2 * 2 * (32 + 31) * 256 * 4
    t = _dummy()
    saved = _native.Saved(0x4000, 0x8000)
    assert lib.sa2_fwd(prob, t, t, t, t, t, t, None, ctypes.c_void_p(0x2000), ctypes.byref(saved), None) == 3
    assert b'256' in lib.sa2_last_error()


def test_argument_validation_happens_before_any_launch(lib):
    good = _native.problem(1, 64, 2, 1, 128, 512, 32, True, 128 ** -0.5)
    t = _dummy()
    lse = ctypes.c_void_p(0x2000)

    def fwd(prob, *tensors, lse_ptr=lse):
        return lib.sa2_fwd(prob, *tensors, None, lse_ptr, None, None)

    assert fwd(None, t, t, t, t, t, t) == 1
    assert fwd(good, None, t, t, t, t, t) == 1
    assert b'q' in lib.sa2_last_error()
    assert fwd(good, t, t, t, t, t, t, lse_ptr=None) == 1
    for field, value, code in [('dim_head', 96, 3), ('causal', 0, 3), ('dtype', 7, 3), ('w1', 0, 2), ('w2', -1, 2),
                               ('seq_len', 0, 2), ('kv_heads', 3, 2), ('batch', 0, 2)]:
        bad = _native.problem(1, 64, 2, 1, 128, 512, 32, True, 128 ** -0.5)
        setattr(bad, field, value)
        assert fwd(bad, t, t, t, t, t, t) == code, field
        assert lib.sa2_last_error() != b''
    assert fwd(good, _dummy(ptr=0x1008), t, t, t, t, t) == 4
    assert fwd(good, t, _dummy(sn=132), t, t, t, t) == 4
    with pytest.raises(_native.Sa2Error) as e:
        _native.check(fwd(good, t, t, _dummy(sh=4), t, t, t))
    assert 'SA2_ERR_ALIGNMENT' in str(e.value) and 'k2' in str(e.value)
    # backward entry points validate the same way
    assert lib.sa2_bwd_delta(good, None, None, t, lse, None) == 1
    need = lib.sa2_bwd_workspace_bytes(good)
    assert need == 2 * 1 * 2 * 2 * 63 * 128 * 4          # 2 tensors, B*H*tiles blocks of 63 fp32 rows
    assert lib.sa2_bwd_workspace_bytes(None) == -1
    # with saved forward partials: half of the partial rows ...
    assert lib.sa2_bwd_workspace_bytes_with_saved(good) == need // 2
    assert lib.sa2_bwd_workspace_bytes_with_saved(None) == -1
    # ... but at least the two fp32 partial results of dk1/dv1 where the key slabs are split over two workgroups
    # each (a grid of two ragged workgroups per CU: the layer shape of benchmark config 5 on 256 CUs)
    layer5 = _native.problem(8, 2048, 8, 4, 64, 512, 32, True, 0.125)
    rows5 = 2 * 8 * 8 * 64 * 63 * 64 * 4
    parts5 = 2 * 2 * 8 * 4 * 2048 * 64 * 4
    assert lib.sa2_bwd_workspace_bytes(layer5) == rows5
    assert lib.sa2_bwd_workspace_bytes_with_saved(layer5) == max(rows5 // 2, parts5) == parts5
    # an even grid of equal workgroups is left alone (config 3: eight workgroups per CU)
    config3 = _native.problem(4, 8192, 8, 8, 128, 512, 32, True, 0.1)
    assert lib.sa2_bwd_workspace_bytes_with_saved(config3) * 2 == lib.sa2_bwd_workspace_bytes(config3)
    assert lib.sa2_bwd_dq_dkv2(good, t, t, t, t, t, t, None, lse, None, t, t, t, lse, need, None) == 1
    assert lib.sa2_bwd_dq_dkv2(good, t, t, t, t, t, t, lse, lse, None, t, t, t, None, need, None) == 1
    assert lib.sa2_bwd_dq_dkv2(good, t, t, t, t, t, t, lse, lse, None, t, t, t, lse, need - 1, None) == 2
    assert lib.sa2_bwd_dq_dkv2(good, t, t, t, t, t, t, lse, lse, None, t, t, _dummy(ptr=0x1004), lse, need, None) == 4
    assert lib.sa2_bwd_dkv1(good, t, t, t, t, t, t, lse, lse, None, t, None) == 1
    assert lib.sa2_bwd(good, t, t, t, t, t, None, None, t, lse, None, lse, t, t, t, t, t, lse, need, None) == 1
    # saved forward partials: sizes, and NULL members are refused
    assert lib.sa2_saved_t_bytes(good) == 1 * 2 * 32 * 64 * 128 * 2
    assert lib.sa2_saved_m_bytes(good) == 1 * 2 * 32 * 64 * 4
    # the partials are kept in whole blocks of 32 rows: a ragged sequence length rounds up
    ragged = _native.problem(1, 65, 2, 2, 128, 16, 32, True, 0.1)
    assert lib.sa2_saved_t_bytes(ragged) == 1 * 2 * 32 * 96 * 128 * 2
    assert lib.sa2_saved_m_bytes(ragged) == 1 * 2 * 32 * 65 * 4
    assert lib.sa2_saved_t_bytes(None) == -1
    assert lib.sa2_fwd(good, t, t, t, t, t, t, None, lse, ctypes.byref(_native.Saved(None, None)), None) == 1
    assert lib.sa2_fwd(good, t, t, t, t, t, t, None, lse, ctypes.byref(_native.Saved(0x1004, 0x2000)), None) == 4


def test_function_rejects_what_the_kernels_do_not_cover():
    q = torch.randn(1, 16, 2, 64)
    with pytest.raises(AssertionError):          # reference: assert all is_cuda (triton_two_simplicial_attention.py:729)
        S.sliding_two_simplicial_attn(q, (q, q), (q, q))
    with pytest.raises(AssertionError):
        S.sliding_two_simplicial_attn(q, (q,), (q, q))
    with pytest.raises(AssertionError):          # head divisibility (triton_two_simplicial_attention.py:1030)
        S.sliding_two_simplicial_attn(torch.randn(1, 16, 3, 64), (q, q), (q, q))


def test_wrapper_checks_head_dimensions_and_dtypes():
    q = torch.randn(1, 16, 2, 64)
    wide = torch.randn(1, 16, 2, 264)
    with pytest.raises(NotImplementedError):     # beyond the kernels' largest head dimension
        S.sliding_two_simplicial_attn(wide, (wide, wide), (wide, wide))
    with pytest.raises(ValueError):              # k2 with a head dimension of its own
        S.sliding_two_simplicial_attn(q, (q, q[..., :32]), (q, q))
    with pytest.raises(ValueError):
        S.sliding_two_simplicial_attn(q, (q, q), (q, q[..., :32]))
    with pytest.raises(TypeError):
        S.sliding_two_simplicial_attn(q.double(), (q.double(),) * 2, (q.double(),) * 2)


def test_module_with_a_value_head_dimension_of_its_own():
    """dim_head_values (simplicial_mha.py:34,56 of the reference) sizes the value part of the
    projection, the value norms and the output projection."""
    m = S.HigherOrderAttention(dim=64, dim_head=16, dim_head_values=8, heads=2, key_value_heads=1, causal=True)
    assert m.to_qkv.weight.shape == (2 * 16 + 2 * 16 + 2 * 8, 64)
    assert m.combine_heads.weight.shape == (64, 2 * 8)
    assert m.v_norms[0].weight.shape == (8,) and m.k_norms[0].weight.shape == (16,)
    assert m(torch.randn(2, 10, 64)).shape == (2, 10, 64)


def test_module_mirrors_reference_constructor_and_parameters():
    m = S.SlidingWindowTwoSimplicialMHA(dim=512, dim_head=64, heads=8)
    sd = m.state_dict()
    assert set(sd) == {'q_norm.weight', 'k_norms.0.weight', 'k_norms.1.weight', 'v_norms.0.weight',
                       'v_norms.1.weight', 'to_qkv.weight', 'combine_heads.weight'}
    assert sd['to_qkv.weight'].shape == (8 * 64 + 2 * 8 * 64 + 2 * 8 * 64, 512)
    assert sd['combine_heads.weight'].shape == (512, 512)
    assert m.attend.keywords == {'w1': 512, 'w2': 32, 'causal': True}
    g = S.SlidingWindowTwoSimplicialMHA(dim=256, dim_head=64, heads=8, key_value_heads=4, w1=128, w2=16,
                                        prenorm=True, postnorm=True, qk_rmsnorm=False)
    assert g.to_qkv.weight.shape == (8 * 64 + 2 * 4 * 64 + 2 * 4 * 64, 256)
    assert {'prenorm.weight', 'postnorm.weight'} <= set(g.state_dict())
    assert g.query_head_groups == 2
    with pytest.raises(AssertionError):
        S.SlidingWindowTwoSimplicialMHA(dim=64, number_key_value_sets=3)
    with pytest.raises(AssertionError):
        S.SlidingWindowTwoSimplicialMHA(dim=64, head_first_dim=True)
    with pytest.raises(AssertionError):
        S.TwoSimplicialMHA(dim=64, number_key_value_sets=2)


def test_alias_module_exposes_reference_names():
    from simplicial_attention_amd import triton_two_simplicial_attention as T
    assert T.sliding_two_simplicial_attn is S.sliding_two_simplicial_attn
    assert T.SlidingWindowTwoSimplicialMHA is S.SlidingWindowTwoSimplicialMHA
    assert T._sliding_two_simplicial_attn.__self__ is S.SlidingTwoSimplicialAttention


def test_module_channel_order_with_oracle_attend():
    """Module plumbing (projection split, '(head, set, d)' channel order, per-head
    RMSNorm on q, k and v, merge) against an explicit restatement with the same weights
    (simplicial_mha.py:110-138 in the reference), using the oracle as `attend`."""
    torch.manual_seed(0)
    dim, heads, kvh, dh, n = 32, 4, 2, 8, 12
    attend = lambda q, k, v: R.sliding_two_simplicial_attn(q, k, v, w1=5, w2=3)
    m = S.HigherOrderAttention(dim, dim_head=dh, heads=heads, key_value_heads=kvh, attend=attend, head_first_dim=False)
    for prm in m.parameters():
        torch.nn.init.normal_(prm, std=0.5)
    x = torch.randn(2, n, dim)
    got = m(x)
    w = m.to_qkv.weight
    proj = x @ w.t()
    q = proj[..., :heads * dh].reshape(2, n, heads, dh)
    k = proj[..., heads * dh:heads * dh + 2 * kvh * dh].reshape(2, n, kvh, 2, dh)
    v = proj[..., heads * dh + 2 * kvh * dh:].reshape(2, n, kvh, 2, dh)
    rms = lambda t, wt: t / t.pow(2).mean(-1, keepdim=True).add(torch.finfo(t.dtype).eps).sqrt() * wt
    q = rms(q, m.q_norm.weight)
    k1, k2 = rms(k[..., 0, :], m.k_norms[0].weight), rms(k[..., 1, :], m.k_norms[1].weight)
    v1, v2 = rms(v[..., 0, :], m.v_norms[0].weight), rms(v[..., 1, :], m.v_norms[1].weight)
    out = R.sliding_two_simplicial_attn(q, (k1, k2), (v1, v2), w1=5, w2=3)
    want = out.reshape(2, n, heads * dh) @ m.combine_heads.weight.t()
    assert torch.allclose(got, want, atol=1e-5)


def test_naive_attend_matches_oracle_restatement():
    g = torch.Generator().manual_seed(1)
    q = torch.randn(2, 4, 10, 8, generator=g)
    k1, k2, v1, v2 = [torch.randn(2, 2, 10, 8, generator=g) for _ in range(4)]
    for causal in (False, True):
        a = S.naive_two_simplicial_attend(q, (k1, k2), (v1, v2), causal=causal)
        b = R.naive_two_simplicial_attend(q, (k1, k2), (v1, v2), causal=causal)
        assert torch.allclose(a, b, atol=1e-6)
    t = torch.randn(1, 16, 512)
    assert S.TwoSimplicialMHA(dim=512, causal=True)(t).shape == t.shape   # tests/test_attn.py:49-55 in the reference


def test_bench_refuses_more_than_one_gpu():
    import subprocess, sys
    r = subprocess.run([sys.executable, os.path.join(ROOT, 'bench.py'), '--gpus', '2'], capture_output=True, text=True)
    assert r.returncode != 0 and 'one GPU' in r.stderr


def test_product_library_reads_no_environment_switches(lib):
    """Switches that skip launches (for kernel timing) exist in the profiling build only: the
    library the package loads must not even contain their names."""
    blob = open(_native.LIB_PATH, 'rb').read()
    for name in (b'SA2_BWD_PASS', b'SA2_BWD_KV1_SPLIT', b'SA2_BWD_QK2_IMPL', b'SA2_BWD_KV1_IMPL'):
        assert name not in blob, name
    prof = open(_native.PROF_LIB_PATH, 'rb').read()
    assert b'SA2_BWD_PASS' in prof


def test_reference_import_paths_resolve_to_this_build():
    """The import lines of the reference's README and tests work unchanged
    (README.md:19, tests/test_triton.py:18, tests/test_attn.py:1-3 of the reference)."""
    from simplicial_attention.triton_two_simplicial_attention import (
        SlidingTwoSimplicialAttention, SlidingWindowTwoSimplicialMHA, sliding_two_simplicial_attn)
    from simplicial_attention import naive_two_simplicial_attend, TwoSimplicialMHA, HigherOrderAttention
    from simplicial_attention.simplicial_attention import naive_two_simplicial_attend as naive2
    from simplicial_attention.simplicial_mha import HigherOrderAttention as HOA
    from simplicial_attention.two_simplicial_transformer import TwoSimplicialTransformer
    assert SlidingWindowTwoSimplicialMHA is S.SlidingWindowTwoSimplicialMHA
    assert SlidingTwoSimplicialAttention is S.SlidingTwoSimplicialAttention
    assert sliding_two_simplicial_attn is S.sliding_two_simplicial_attn
    assert naive2 is naive_two_simplicial_attend is S.naive_two_simplicial_attend
    assert HOA is HigherOrderAttention is S.HigherOrderAttention and TwoSimplicialMHA is S.TwoSimplicialMHA
    attn = SlidingWindowTwoSimplicialMHA(dim=512, dim_head=64, heads=8)
    assert isinstance(attn, HigherOrderAttention) and TwoSimplicialTransformer is not None


def test_saved_partials_budget_is_global_per_device(monkeypatch):
    """The forward keeps its per-offset partials only within a per-call cap and a per-device total; buffers that
    die give their bytes back.  The rule looks at sizes only (never at the memory that happens to be free), so
    which backward path a layer takes does not depend on what else the allocator holds."""
    from simplicial_attention_amd.two_simplicial_attention import _PartialsBudget
    monkeypatch.delenv('SA2_SAVE_PARTIALS_MAX_GIB', raising=False)
    monkeypatch.delenv('SA2_SAVE_PARTIALS_TOTAL_FRACTION', raising=False)
    gib = 1 << 30
    budget = _PartialsBudget()
    total = 288 * gib
    assert not budget.admit(0, 'cuda:0', total)
    assert not budget.admit(17 * gib, 'cuda:0', total)   # per-call cap (16 GiB)
    for _ in range(4):
        assert budget.admit(16 * gib, 'cuda:0', total)   # 64 GiB alive
    assert budget.admit(8 * gib, 'cuda:0', total)        # 72 GiB = a quarter of the device
    assert not budget.admit(1 * gib, 'cuda:0', total)    # the total is spent ...
    assert budget.admit(1 * gib, 'cuda:1', total)        # ... on that device only
    budget.release(16 * gib, 0)
    assert budget.admit(16 * gib, 'cuda:0', total)
    monkeypatch.setenv('SA2_SAVE_PARTIALS_MAX_GIB', '0')
    assert not _PartialsBudget().admit(1, 'cuda:0', total)
    monkeypatch.setenv('SA2_SAVE_PARTIALS_MAX_GIB', '16')
    monkeypatch.setenv('SA2_SAVE_PARTIALS_TOTAL_FRACTION', '0.01')
    assert not _PartialsBudget().admit(3 * gib, 'cuda:0', total)


def test_signed_determinant_is_the_triple_product_of_channel_triples():
    """simplicial_attention.py:36-76: every triple of channels contributes det[q; k1; k2]; pinned against
    torch.linalg.det, with left-over channels contributing their plain trilinear product."""
    from simplicial_attention_amd.naive import signed_determinant, naive_two_simplicial_attend
    g = torch.Generator().manual_seed(5)
    b, h, n, d = 1, 2, 5, 8                      # two triples and two left-over channels
    q, k1, k2 = (torch.randn(b, h, n, d, generator=g, dtype=torch.float64) for _ in range(3))
    got = signed_determinant(q, k1, k2)
    want = torch.zeros(b, h, n, n, n, dtype=torch.float64)
    for i in range(n):
        for j in range(n):
            for k in range(n):
                for t in range(d // 3):
                    m = torch.stack([q[:, :, i, 3 * t:3 * t + 3], k1[:, :, j, 3 * t:3 * t + 3], k2[:, :, k, 3 * t:3 * t + 3]], dim=-2)
                    want[:, :, i, j, k] += torch.linalg.det(m)
                want[:, :, i, j, k] += (q[:, :, i, 6:] * k1[:, :, j, 6:] * k2[:, :, k, 6:]).sum(-1)
    assert torch.allclose(got, want, atol=1e-10)
    # antisymmetric in the two key sets on the full triples
    q6, a6, b6 = q[..., :6], k1[..., :6], k2[..., :6]
    assert torch.allclose(signed_determinant(q6, a6, b6), -signed_determinant(q6, b6, a6).transpose(-1, -2), atol=1e-10)
    v1, v2 = (torch.randn(b, h, n, d, generator=g, dtype=torch.float64) for _ in range(2))
    out = naive_two_simplicial_attend(q, (k1, k2), (v1, v2), causal=True, use_signed_determinant=True)
    assert out.shape == (b, h, n, d) and torch.isfinite(out).all()


def test_nth_order_attend_special_cases():
    """simplicial_attention.py:131-198: one key/value set is ordinary attention (pinned against
    scaled_dot_product_attention), two sets are the 2-simplicial attend, three sets are pinned by loops."""
    from simplicial_attention_amd.naive import nth_order_attend, naive_two_simplicial_attend
    g = torch.Generator().manual_seed(6)
    b, h, hk, n, d = 2, 4, 2, 6, 8
    q = torch.randn(b, h, n, d, generator=g, dtype=torch.float64)
    ks = [torch.randn(b, hk, n, d, generator=g, dtype=torch.float64) for _ in range(3)]
    vs = [torch.randn(b, hk, n, d, generator=g, dtype=torch.float64) for _ in range(3)]
    for causal in (False, True):
        one = nth_order_attend(q, ks[:1], vs[:1], causal=causal)
        sdpa = torch.nn.functional.scaled_dot_product_attention(q, ks[0].repeat_interleave(2, 1), vs[0].repeat_interleave(2, 1), is_causal=causal)
        assert torch.allclose(one, sdpa, atol=1e-10)
        two = nth_order_attend(q, ks[:2], vs[:2], causal=causal)
        assert torch.allclose(two, naive_two_simplicial_attend(q, ks[:2], vs[:2], causal=causal), atol=1e-10)
    three = nth_order_attend(q, ks, vs)
    want = torch.zeros_like(three)
    for bi in range(b):
        for hi in range(h):
            kh = hi // 2
            for i in range(n):
                logits = torch.einsum('d,jd,kd,ld->jkl', q[bi, hi, i] * d ** -0.5, ks[0][bi, kh], ks[1][bi, kh], ks[2][bi, kh])
                w = logits.flatten().softmax(0).view_as(logits)
                want[bi, hi, i] = torch.einsum('jkl,jd,kd,ld->d', w, vs[0][bi, kh], vs[1][bi, kh], vs[2][bi, kh])
    assert torch.allclose(three, want, atol=1e-10)


def test_module_with_three_key_value_sets_uses_the_nth_order_attend():
    import simplicial_attention_amd as S
    torch.manual_seed(0)
    m = S.HigherOrderAttention(dim=32, dim_head=8, heads=2, number_key_value_sets=3)
    assert m.attend is S.nth_order_attend
    out = m(torch.randn(1, 5, 32))
    assert out.shape == (1, 5, 32) and torch.isfinite(out).all()
    with pytest.raises(AssertionError):
        S.HigherOrderAttention(dim=32, dim_head=8, heads=2, number_key_value_sets=3, causal=True)
