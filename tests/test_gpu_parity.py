"""GPU parity: the HIP path (through the C ABI of libsa2.so) against the CPU oracle
on the same seeded, bf16-rounded inputs, for the output and all five input gradients.
Every shape runs with both input distributions and the tolerance stated for each
(see tests/parity_util.py)."""
import pytest
import torch

from oracle import reference_attend as R
from tests import parity_util as U

pytestmark = pytest.mark.gpu

CASES = [
    # b, n, hq, hk, d, w1, w2
    (1, 32, 1, 1, 128, 512, 32),      # windows >= N: pure causal (reference test_triton.py script, N=32)
    (1, 64, 1, 1, 64, 16, 4),
    (2, 128, 4, 4, 64, 64, 32),       # shape of the reference's tests/test_triton.py:68-83
    (1, 128, 2, 2, 128, 64, 32),
    (2, 200, 4, 2, 128, 48, 8),       # ragged N, grouped heads
    (1, 300, 2, 1, 64, 100, 33),      # windows not multiples of 32, w2 > 32
    (1, 640, 2, 2, 128, 512, 32),     # default windows, D = 128
    (1, 1000, 2, 2, 64, 512, 32),     # ragged N with the default windows
    (1, 150, 2, 2, 128, 40, 5),       # odd number of offsets: the last offset pair of a step is half empty
    (1, 260, 2, 1, 128, 70, 64),      # second window of two offset blocks, D = 128
    (1, 200, 2, 2, 64, 48, 65),       # second windows beyond 64 (the reference's backward stops at 32,
    (1, 330, 2, 1, 128, 96, 100),     #   triton_two_simplicial_attention.py:586): offset rounds, offset blocks
    (2, 160, 2, 2, 128, 160, 128),    # both windows >= N: full causal over three offset blocks
    (1, 1, 1, 1, 128, 512, 32),       # a single row
    (1, 17, 2, 1, 64, 512, 32),       # less than one tile
    (2, 31, 4, 2, 128, 8, 32),        # less than one tile, second window wider than the sequence
    (1, 128, 4, 4, 32, 128, 128),     # head dimension 32 (native instance): shape of the reference's CPU-runnable case
    (2, 333, 4, 2, 32, 100, 32),      # head dimension 32, ragged N, grouped heads
    (1, 200, 2, 1, 32, 48, 70),       # head dimension 32, several offset blocks
    (1, 19, 2, 2, 32, 512, 32),       # head dimension 32, less than one tile
    (1, 128, 2, 2, 256, 64, 32),      # head dimension 256 (kernels of their own: the waves of a workgroup split the head dimension)
    (2, 300, 4, 2, 256, 100, 40),     # head dimension 256, ragged N, grouped heads, second window beyond 32
    (1, 45, 2, 1, 256, 512, 32),      # head dimension 256, windows wider than the sequence
    (1, 1, 1, 1, 256, 512, 32),       # head dimension 256, a single row
]


@pytest.mark.parametrize('unit_variance', [False, True], ids=['std_rsqrt_d', 'std_1'])
@pytest.mark.parametrize('b,n,hq,hk,d,w1,w2', CASES)
def test_fwd_bwd_matches_oracle(b, n, hq, hk, d, w1, w2, unit_variance):
    print(f'\ncase b={b} n={n} hq={hq} hk={hk} d={d} w1={w1} w2={w2} unit_variance={unit_variance}', flush=True)
    ins = U.make_inputs(b, n, hq, hk, d, seed=n + d + w1, std=1.0 if unit_variance else d ** -0.5)
    ref_out, _, ref_grads = U.oracle_fwd_bwd(*ins, w1, w2)
    out, grads = U.hip_fwd_bwd(*ins, w1, w2)
    U.check_all(out, grads, ref_out, ref_grads, unit_variance=unit_variance)


def _random_shapes(count, seed=1234, dims=(32, 64, 128)):
    import random
    rng = random.Random(seed)
    shapes = []
    for _ in range(count):
        d = rng.choice(list(dims))
        hk = rng.choice([1, 2])
        hq = hk * rng.choice([1, 2])
        n = rng.choice([rng.randint(1, 40), rng.randint(33, 130), rng.randint(131, 420)])
        w1 = rng.choice([rng.randint(1, 40), rng.randint(30, 140), rng.randint(100, 600)])
        w2 = rng.choice([rng.randint(1, 9), rng.randint(8, 33), rng.randint(30, 80)])
        shapes.append((rng.choice([1, 2]), n, hq, hk, d, w1, w2))
    return shapes


@pytest.mark.parametrize('b,n,hq,hk,d,w1,w2', _random_shapes(24))
def test_seeded_random_shapes(b, n, hq, hk, d, w1, w2):
    """A seeded draw of sequence lengths, windows, head counts and head dimensions (ragged tiles, windows
    shorter and longer than the sequence, one to ten offset rounds, grouped heads)."""
    print(f'\ncase b={b} n={n} hq={hq} hk={hk} d={d} w1={w1} w2={w2}', flush=True)
    ins = U.make_inputs(b, n, hq, hk, d, seed=n * 7 + w1 * 3 + w2, std=d ** -0.5)
    ref_out, _, ref_grads = U.oracle_fwd_bwd(*ins, w1, w2)
    out, grads = U.hip_fwd_bwd(*ins, w1, w2)
    U.check_all(out, grads, ref_out, ref_grads)


@pytest.mark.parametrize('b,n,hq,hk,d,w1,w2', _random_shapes(10, seed=4321, dims=(256,)))
def test_seeded_random_shapes_head_dimension_256(b, n, hq, hk, d, w1, w2):
    """The same draw for the kernels of head dimension 256."""
    print(f'\ncase b={b} n={n} hq={hq} hk={hk} d={d} w1={w1} w2={w2}', flush=True)
    ins = U.make_inputs(b, n, hq, hk, d, seed=n * 7 + w1 * 3 + w2, std=d ** -0.5)
    ref_out, _, ref_grads = U.oracle_fwd_bwd(*ins, w1, w2)
    out, grads = U.hip_fwd_bwd(*ins, w1, w2)
    U.check_all(out, grads, ref_out, ref_grads)


@pytest.mark.parametrize('d', [128, 256])
def test_large_and_drifting_logits(d):
    """Logits that grow along the sequence by far more than 2^64 per window: exercises
    the paths of the forward that move the softmax reference point while accumulators
    hold data.  q and k2 hold powers of two and the softmax scale is chosen so that
    scale * log2(e) = 2^-4, so the bf16 operand q * k2 * scale * log2(e) that the kernels feed
    to the MFMA is exact and the large logits carry no operand-rounding error (which would
    otherwise dominate any comparison at this scale, for the reference's kernels as well:
    they round q * k1 * scale to bf16, triton_two_simplicial_attention.py:150-152, 182)."""
    import math
    from simplicial_attention_amd import SlidingTwoSimplicialAttention
    b, n, h, w1, w2 = 1, 256, 2, 96, 16
    scale = 2.0 ** -4 / math.log2(math.e)
    g = torch.Generator().manual_seed(21)
    q = torch.pow(2.0, torch.randint(-1, 2, (b, n, h, d), generator=g).float()).bfloat16()
    k2 = torch.pow(2.0, torch.randint(0, 2, (b, n, h, d), generator=g).float()).bfloat16()
    ramp = torch.linspace(0.2, 12.0, n).view(1, n, 1, 1)
    k1 = (torch.randn(b, n, h, d, generator=g).abs() * ramp * 2.0).bfloat16()
    v1, v2, dout = [torch.randn(b, n, h, d, generator=g).bfloat16() for _ in range(3)]
    f64 = lambda t: t.double()
    ref_out, ref_lse, ref_grads = R.windowed_banded_fwd_bwd(f64(q), f64(k1), f64(k2), f64(v1), f64(v2), f64(dout), w1, w2, scale=scale)
    assert float(ref_lse.max() - ref_lse.min()) > 100.0       # natural-log units
    ts = [t.cuda().requires_grad_(True) for t in (q, k1, k2, v1, v2)]
    out = SlidingTwoSimplicialAttention.apply(*ts, w1, w2, True, scale)
    grads = torch.autograd.grad(out, ts, dout.cuda())
    assert torch.isfinite(out.float()).all()
    row = U.compare('out', out, ref_out)
    assert row['bad'] == 0 and row['rel_fro'] <= 1e-2, row
    # gradients reach magnitudes of 30-60 here (k1 is scaled up to 24x): relative check only
    for name, got, ref in zip(U.NAMES[1:], grads, ref_grads):
        row = U.compare(name, got, ref)
        print('  ', row, flush=True)
        assert row['rel_fro'] <= 3e-2, row


@pytest.mark.parametrize('std', [0.5, 1.0])
def test_degenerate_windows_attend_only_self(std):
    """w1 = w2 = 1: every row attends (i, i) only, so out_i = v1_i * v2_i and
    dq = dk1 = dk2 = 0 exactly.  The kernels form dS = P (dP - delta) from a bf16 MFMA
    dP and an fp32 delta, which agree to the bf16 rounding of the operand do * v2 only:
    what comes back instead of zero is that rounding, about 1e-2 at std 0.5 (inside the
    build criterion) and 3e-2 at std 1.0 (inside the reference's gradient tolerance of 5e-2,
    tests/test_triton.py:111-115, outside the build criterion: judged by the former).
    Splitting do * v2 into two bf16 operands would remove it at the price of a second dP
    chain (+ 8 of 24 / 32 MFMAs per step in the two backward kernels, 32 more registers in
    one that has none, an LDS tile in the other); an error model of the backward's
    roundings shows that it would lower the gradients' relative error by a fifth at most
    in non-degenerate cases, where the rounding of q * k2 (which the reference shares,
    triton_two_simplicial_attention.py:150-152) dominates."""
    ins = U.make_inputs(1, 100, 2, 2, 128, seed=3, std=std)
    ref_out, _, ref_grads = U.oracle_fwd_bwd(*ins, 1, 1)
    out, grads = U.hip_fwd_bwd(*ins, 1, 1)
    assert float(ref_grads[0].abs().max()) < 1e-5
    want = ins[3].float() * ins[4].float()
    assert torch.allclose(out.float().cpu(), want, atol=1e-2 * max(1.0, 4 * std * std), rtol=1e-2)
    U.check_all(out, grads, ref_out, ref_grads, rel_fro_limit=float('inf'), unit_variance=True,
                reference_atol_only=std == 1.0)


def test_lse_matches_oracle():
    from simplicial_attention_amd import _native
    b, n, h, d, w1, w2 = 1, 256, 2, 128, 96, 16
    q, k1, k2, v1, v2, _ = U.make_inputs(b, n, h, h, d, seed=5)
    ts = [t.cuda() for t in (q, k1, k2, v1, v2)]
    out = torch.empty_like(ts[0])
    lse = torch.empty(b, h, n, dtype=torch.float32, device='cuda')
    lib = _native.load()
    prob = _native.problem(b, n, h, h, d, w1, w2, True, d ** -0.5)
    _native.check(lib.sa2_fwd(prob, *(_native.tensor_arg(t) for t in (*ts, out)), None, lse.data_ptr(), None,
                              torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    from oracle import reference_attend as R
    _, ref = R.windowed_banded(*[t.float() for t in (q, k1, k2, v1, v2)], w1, w2)
    assert torch.allclose(lse.cpu(), ref, atol=2e-2, rtol=1e-2)


@pytest.mark.parametrize('shape', [(2, 320, 4, 2, 128, 96, 16), (1, 200, 2, 2, 64, 64, 32), (1, 200, 2, 1, 32, 64, 32)])
def test_backward_that_recomputes_instead_of_using_saved_partials(shape, monkeypatch):
    """SA2_SAVE_PARTIALS_MAX_GIB=0: the forward keeps no per-offset T and dV2 comes from
    the recomputing pass (what the reference does)."""
    monkeypatch.setenv('SA2_SAVE_PARTIALS_MAX_GIB', '0')
    b, n, hq, hk, d, w1, w2 = shape
    ins = U.make_inputs(b, n, hq, hk, d, seed=23, std=d ** -0.5)
    ref_out, _, ref_grads = U.oracle_fwd_bwd(*ins, w1, w2)
    out, grads = U.hip_fwd_bwd(*ins, w1, w2)
    U.check_all(out, grads, ref_out, ref_grads)


@pytest.mark.parametrize('dtype,dqk,dv,n,w1,w2', [
    (torch.float32, 32, 32, 128, 128, 64),     # head size and dtype of the reference's CPU-runnable case
    (torch.bfloat16, 64, 32, 200, 64, 16),     # value heads narrower than query/key heads
    (torch.float16, 48, 128, 150, 40, 8),      # neither 64 nor 128; value heads wider
    (torch.bfloat16, 96, 96, 100, 512, 32),
    (torch.bfloat16, 192, 192, 100, 64, 32),   # padded to 256
    (torch.float32, 256, 160, 70, 512, 8),     # query/key heads of 256, narrower value heads
])
def test_other_head_dimensions_and_dtypes(dtype, dqk, dv, n, w1, w2):
    """Head dimensions other than 32/64/128 (and the native 32), a value head dimension of its own, and float16 /
    float32 tensors: the functional wrapper pads and casts around the bf16 kernels; output
    and gradients come back in the caller's dtype and shapes.  The oracle works on the
    bf16-rounded values with the scale of the true query/key dimension."""
    from simplicial_attention_amd import sliding_two_simplicial_attn
    b, hq, hk = 1, 4, 2
    g = torch.Generator(device='cpu').manual_seed(dqk + dv)
    rnd = lambda h, d: torch.randn(b, n, h, d, generator=g).bfloat16()
    q, k1, k2 = rnd(hq, dqk), rnd(hk, dqk), rnd(hk, dqk)
    v1, v2, dout = rnd(hk, dv), rnd(hk, dv), rnd(hq, dv)
    ref_out, _, ref_grads = U.oracle_fwd_bwd(q, k1, k2, v1, v2, dout, w1, w2)
    ts = [t.to(dtype).cuda().requires_grad_(True) for t in (q, k1, k2, v1, v2)]
    out = sliding_two_simplicial_attn(ts[0], (ts[1], ts[2]), (ts[3], ts[4]), w1=w1, w2=w2)
    assert out.dtype is dtype and out.shape == (b, n, hq, dv)
    grads = torch.autograd.grad(out, ts, dout.to(dtype).cuda())
    for got, leaf in zip(grads, ts):
        assert got.dtype is dtype and got.shape == leaf.shape
    U.check_all(out, grads, ref_out, ref_grads, unit_variance=True)


@pytest.mark.parametrize('d', [128, 256])
def test_backward_is_deterministic(d):
    ins = U.make_inputs(1, 384, 2, 1, d, seed=11)
    first = U.hip_fwd_bwd(*ins, 128, 32)
    for _ in range(2):
        again = U.hip_fwd_bwd(*ins, 128, 32)
        assert torch.equal(first[0], again[0])
        for a, b_ in zip(first[1], again[1]):
            assert torch.equal(a, b_)


def test_strided_views_need_no_copy():
    """q, k1, k2, v1, v2 as interleaved views of one packed (b, n, 5h, d) buffer and a dout view
    with padded rows: the kernels take the strides as they are (no .contiguous() copy)."""
    from simplicial_attention_amd import sliding_two_simplicial_attn
    b, n, h, d, w1, w2 = 2, 300, 2, 128, 128, 16
    q, k1, k2, v1, v2, dout = U.make_inputs(b, n, h, h, d, seed=31, std=d ** -0.5)
    packed = torch.stack((q, k1, k2, v1, v2), dim=3).reshape(b, n, h * 5, d).cuda()      # channel (head, tensor)
    views = [packed.view(b, n, h, 5, d)[:, :, :, x] for x in range(5)]
    assert not views[0].is_contiguous()
    dpad = torch.zeros(b, n, h, d + 16, dtype=torch.bfloat16, device='cuda')
    dpad[..., :d] = dout.cuda()
    leaves = [v.detach().clone().requires_grad_(True) for v in views]                  # contiguous run
    out_c = sliding_two_simplicial_attn(leaves[0], (leaves[1], leaves[2]), (leaves[3], leaves[4]), w1=w1, w2=w2)
    grads_c = torch.autograd.grad(out_c, leaves, dout.cuda())
    pk = packed.clone().requires_grad_(True)
    vs = [pk.view(b, n, h, 5, d)[:, :, :, x] for x in range(5)]
    out_s = sliding_two_simplicial_attn(vs[0], (vs[1], vs[2]), (vs[3], vs[4]), w1=w1, w2=w2)
    (gpk,) = torch.autograd.grad(out_s, pk, dpad[..., :d])
    torch.cuda.synchronize()
    assert torch.equal(out_s, out_c)
    for x in range(5):
        assert torch.equal(gpk.view(b, n, h, 5, d)[:, :, :, x], grads_c[x])


def test_each_backward_entry_point_against_the_oracle():
    """sa2_bwd_delta, sa2_bwd_dq_dkv2 (with and without the forward's saved partials) and
    sa2_bwd_dkv1 called one by one through the C ABI, each output against the CPU oracle."""
    from simplicial_attention_amd import _native
    lib = _native.load()
    arg = _native.tensor_arg
    b, n, hq, hk, d, w1, w2 = 2, 300, 4, 2, 128, 100, 40
    ins = U.make_inputs(b, n, hq, hk, d, seed=77, std=d ** -0.5)
    ref_out, ref_lse, ref_grads = U.oracle_fwd_bwd(*ins, w1, w2)
    q, k1, k2, v1, v2, dout = (t.cuda() for t in ins)
    prob = _native.problem(b, n, hq, hk, d, w1, w2, True, d ** -0.5)
    sh = torch.cuda.current_stream().cuda_stream
    out, res = torch.empty_like(q), torch.empty_like(q)
    lse = torch.empty(b, hq, n, dtype=torch.float32, device='cuda')
    t_save = torch.empty(lib.sa2_saved_t_bytes(prob), dtype=torch.uint8, device='cuda')
    m_save = torch.empty(lib.sa2_saved_m_bytes(prob), dtype=torch.uint8, device='cuda')
    saved = _native.saved_arg(t_save, m_save)
    _native.check(lib.sa2_fwd(prob, arg(q), arg(k1), arg(k2), arg(v1), arg(v2), arg(out), arg(res), lse.data_ptr(), saved, sh))
    # delta = sum_d out * dout
    delta = torch.full_like(lse, float('nan'))
    _native.check(lib.sa2_bwd_delta(prob, arg(out), arg(res), arg(dout), delta.data_ptr(), sh))
    torch.cuda.synchronize()
    want_delta = (ref_out * ins[5].float()).sum(-1).transpose(1, 2)                 # (b, h, n)
    assert torch.allclose(delta.cpu(), want_delta, atol=2e-2, rtol=1e-2)
    assert torch.allclose(lse.cpu(), ref_lse, atol=2e-2, rtol=1e-2)
    ws_bytes = lib.sa2_bwd_workspace_bytes(prob)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device='cuda')
    for use_saved in (True, False):
        dq = torch.full_like(q, float('nan'))
        dk2, dv2 = torch.full_like(k2, float('nan')), torch.full_like(v2, float('nan'))
        _native.check(lib.sa2_bwd_dq_dkv2(prob, arg(q), arg(k1), arg(k2), arg(v1), arg(v2), arg(dout), lse.data_ptr(),
                                          delta.data_ptr(), saved if use_saved else None, arg(dq), arg(dk2), arg(dv2),
                                          ws.data_ptr(), ws_bytes, sh))
        torch.cuda.synchronize()
        for name, got, ref in (('dq', dq, ref_grads[0]), ('dk2', dk2, ref_grads[2]), ('dv2', dv2, ref_grads[4])):
            row = U.compare(name, got, ref)
            print('  ', use_saved, row, flush=True)
            assert row['bad'] == 0 and row['rel_fro'] <= 1e-2, (use_saved, row)
    dk1, dv1 = torch.full_like(k1, float('nan')), torch.full_like(v1, float('nan'))
    _native.check(lib.sa2_bwd_dkv1(prob, arg(q), arg(k1), arg(k2), arg(v1), arg(v2), arg(dout), lse.data_ptr(), delta.data_ptr(),
                                   arg(dk1), arg(dv1), sh))
    torch.cuda.synchronize()
    for name, got, ref in (('dk1', dk1, ref_grads[1]), ('dv1', dv1, ref_grads[3])):
        row = U.compare(name, got, ref)
        print('  ', row, flush=True)
        assert row['bad'] == 0 and row['rel_fro'] <= 1e-2, row
    # the whole backward in one call runs the same kernels (this grid is too small for split key slabs)
    delta2 = torch.empty_like(lse)
    dq2 = torch.full_like(q, float('nan'))
    g2 = [torch.full_like(k1, float('nan')) for _ in range(4)]
    _native.check(lib.sa2_bwd(prob, arg(q), arg(k1), arg(k2), arg(v1), arg(v2), arg(out), arg(res), arg(dout), lse.data_ptr(), None,
                              delta2.data_ptr(), arg(dq2), arg(g2[0]), arg(g2[1]), arg(g2[2]), arg(g2[3]), ws.data_ptr(), ws_bytes, sh))
    torch.cuda.synchronize()
    assert torch.equal(dq2, dq) and torch.equal(g2[1], dk2) and torch.equal(g2[3], dv2)
    assert torch.equal(g2[0], dk1) and torch.equal(g2[2], dv1)


def test_head_dimension_256_entry_points_one_by_one():
    """Head dimension 256 through every entry point of the C ABI: the forward without saved partials (its kernels keep
    none), delta, sa2_bwd_dq_dkv2 on a NaN-filled workspace, sa2_bwd_dkv1, then sa2_bwd and sa2_bwd_noalloc, which must
    give the same bits."""
    from simplicial_attention_amd import _native
    lib = _native.load()
    arg = _native.tensor_arg
    b, n, hq, hk, d, w1, w2 = 2, 210, 4, 2, 256, 70, 20
    ins = U.make_inputs(b, n, hq, hk, d, seed=91, std=d ** -0.5)
    ref_out, ref_lse, ref_grads = U.oracle_fwd_bwd(*ins, w1, w2)
    q, k1, k2, v1, v2, dout = (t.cuda() for t in ins)
    prob = _native.problem(b, n, hq, hk, d, w1, w2, True, d ** -0.5)
    sh = torch.cuda.current_stream().cuda_stream
    out, res = torch.full_like(q, float('nan')), torch.full_like(q, float('nan'))
    lse = torch.full((b, hq, n), float('nan'), dtype=torch.float32, device='cuda')
    _native.check(lib.sa2_fwd(prob, arg(q), arg(k1), arg(k2), arg(v1), arg(v2), arg(out), arg(res), lse.data_ptr(), None, sh))
    delta = torch.full_like(lse, float('nan'))
    _native.check(lib.sa2_bwd_delta(prob, arg(out), arg(res), arg(dout), delta.data_ptr(), sh))
    torch.cuda.synchronize()
    assert U.compare('out', out, ref_out)['bad'] == 0
    assert torch.allclose(lse.cpu(), ref_lse, atol=2e-2, rtol=1e-2)
    assert torch.allclose(delta.cpu(), (ref_out * ins[5].float()).sum(-1).transpose(1, 2), atol=2e-2, rtol=1e-2)
    ws_bytes = lib.sa2_bwd_workspace_bytes(prob)
    ws = torch.full((ws_bytes,), 0xFF, dtype=torch.uint8, device='cuda')
    dq, dk2, dv2 = torch.full_like(q, float('nan')), torch.full_like(k2, float('nan')), torch.full_like(v2, float('nan'))
    _native.check(lib.sa2_bwd_dq_dkv2(prob, arg(q), arg(k1), arg(k2), arg(v1), arg(v2), arg(dout), lse.data_ptr(), delta.data_ptr(),
                                      None, arg(dq), arg(dk2), arg(dv2), ws.data_ptr(), ws_bytes, sh))
    dk1, dv1 = torch.full_like(k1, float('nan')), torch.full_like(v1, float('nan'))
    _native.check(lib.sa2_bwd_dkv1(prob, arg(q), arg(k1), arg(k2), arg(v1), arg(v2), arg(dout), lse.data_ptr(), delta.data_ptr(),
                                   arg(dk1), arg(dv1), sh))
    torch.cuda.synchronize()
    for name, got, ref in zip(U.NAMES[1:], (dq, dk1, dk2, dv1, dv2), ref_grads):
        row = U.compare(name, got, ref)
        print('  ', row, flush=True)
        assert row['bad'] == 0 and row['rel_fro'] <= 1e-2, row
    for entry in ('sa2_bwd', 'sa2_bwd_noalloc'):
        g = [torch.full_like(q, float('nan'))] + [torch.full_like(k1, float('nan')) for _ in range(4)]
        if entry == 'sa2_bwd':
            ws.fill_(0xFF)
            delta2 = torch.full_like(lse, float('nan'))
            _native.check(lib.sa2_bwd(prob, arg(q), arg(k1), arg(k2), arg(v1), arg(v2), arg(out), arg(res), arg(dout), lse.data_ptr(), None,
                                      delta2.data_ptr(), *(arg(t) for t in g), ws.data_ptr(), ws_bytes, sh))
        else:
            assert lib.sa2_bwd_noalloc_scratch_bytes(prob) <= 64 << 20
            _native.check(lib.sa2_bwd_noalloc(prob, arg(q), arg(k1), arg(k2), arg(v1), arg(v2), arg(out), arg(res), arg(dout), lse.data_ptr(),
                                              None, *(arg(t) for t in g), sh))
        torch.cuda.synchronize()
        for got, want in zip(g, (dq, dk1, dk2, dv1, dv2)):
            assert torch.equal(got, want), entry


@pytest.mark.gpu
@pytest.mark.parametrize('n', [1024, 1040])
@pytest.mark.parametrize('d', [32, 64, 128])
def test_split_key_slabs_against_the_oracle_and_single_workgroups(d, n):
    """A grid of one to four dK1/dV1 workgroups per CU on a short sequence: sa2_bwd gives every key slab to two
    workgroups (half of the slab's query tiles each) and adds their fp32 partial results; sa2_bwd_dkv1, which has
    no workspace, keeps one workgroup per slab.  Both against the oracle, and against each other to one rounding.
    n = 1040 ends on a slab of 16 rows with a single query tile: its second workgroup has nothing to walk and only
    writes the zeros that the combine kernel adds.  The workspace starts as NaN, so a partial row that no workgroup
    wrote would show."""
    from simplicial_attention_amd import _native
    lib = _native.load()
    arg = _native.tensor_arg
    b, hq, hk, w1, w2 = 3, 12, 12, 64, 8
    prob = _native.problem(b, n, hq, hk, d, w1, w2, True, d ** -0.5)
    parts = 2 * 2 * b * hk * n * d * 4
    assert lib.sa2_bwd_workspace_bytes_with_saved(prob) == parts, 'the split rule does not apply at this size'
    ins = U.make_inputs(b, n, hq, hk, d, seed=5, std=d ** -0.5)
    _, _, ref_grads = U.oracle_fwd_bwd(*ins, w1, w2)
    q, k1, k2, v1, v2, dout = (t.cuda() for t in ins)
    sh = torch.cuda.current_stream().cuda_stream
    out, res = torch.empty_like(q), torch.empty_like(q)
    lse = torch.empty(b, hq, n, dtype=torch.float32, device='cuda')
    _native.check(lib.sa2_fwd(prob, arg(q), arg(k1), arg(k2), arg(v1), arg(v2), arg(out), arg(res), lse.data_ptr(), None, sh))
    delta = torch.empty_like(lse)
    ws_bytes = lib.sa2_bwd_workspace_bytes(prob)
    ws = torch.full((ws_bytes,), 0xFF, dtype=torch.uint8, device='cuda')       # fp32 NaN everywhere
    dq = torch.full_like(q, float('nan'))
    g = [torch.full_like(k1, float('nan')) for _ in range(4)]
    _native.check(lib.sa2_bwd(prob, arg(q), arg(k1), arg(k2), arg(v1), arg(v2), arg(out), arg(res), arg(dout), lse.data_ptr(), None,
                              delta.data_ptr(), arg(dq), arg(g[0]), arg(g[1]), arg(g[2]), arg(g[3]), ws.data_ptr(), ws_bytes, sh))
    one = [torch.full_like(k1, float('nan')) for _ in range(2)]
    _native.check(lib.sa2_bwd_dkv1(prob, arg(q), arg(k1), arg(k2), arg(v1), arg(v2), arg(dout), lse.data_ptr(), delta.data_ptr(),
                                   arg(one[0]), arg(one[1]), sh))
    torch.cuda.synchronize()
    for name, got, single, ref in (('dk1', g[0], one[0], ref_grads[1]), ('dv1', g[2], one[1], ref_grads[3])):
        for label, t in (('in parts', got), ('single', single)):
            row = U.compare(name, t, ref)
            print('  ', label, row, flush=True)
            assert row['bad'] == 0 and row['rel_fro'] <= 1e-2, (label, row)
        diff = (got.float() - single.float()).abs()
        assert float((diff / single.float().abs().clamp_min(1e-3)).max()) <= 2 ** -7, name     # one bf16 rounding
    for name, got, ref in (('dq', dq, ref_grads[0]), ('dk2', g[1], ref_grads[2]), ('dv2', g[3], ref_grads[4])):
        row = U.compare(name, got, ref)
        assert row['bad'] == 0 and row['rel_fro'] <= 1e-2, row
