"""The backward entry point that brings its own scratch (sa2_bwd_noalloc) against sa2_bwd with
caller-owned buffers: same kernels, so every gradient must be bit-identical.  Two calls in a row,
the second on a smaller problem (the scratch keeps the first call's contents)."""
import pytest
import torch

from simplicial_attention_amd import _native
from tests import parity_util as U

pytestmark = pytest.mark.gpu


def _backward_both_ways(b, n, hq, hk, d, w1, w2, seed, with_saved):
    lib = _native.load()
    arg = _native.tensor_arg
    q, k1, k2, v1, v2, dout = (t.cuda() for t in U.make_inputs(b, n, hq, hk, d, seed=seed, std=d ** -0.5))
    prob = _native.problem(b, n, hq, hk, d, w1, w2, True, d ** -0.5)
    out, res = torch.empty_like(q), torch.empty_like(q)
    lse = torch.empty(b, hq, n, dtype=torch.float32, device='cuda')
    saved = t_save = m_save = None
    if with_saved:
        t_save = torch.empty(lib.sa2_saved_t_bytes(prob), dtype=torch.uint8, device='cuda')
        m_save = torch.empty(lib.sa2_saved_m_bytes(prob), dtype=torch.uint8, device='cuda')
        saved = _native.saved_arg(t_save, m_save)
    sh = torch.cuda.current_stream().cuda_stream
    _native.check(lib.sa2_fwd(prob, arg(q), arg(k1), arg(k2), arg(v1), arg(v2), arg(out), arg(res), lse.data_ptr(), saved, sh))

    def grads():
        return [torch.full_like(q, float('nan'))] + [torch.full_like(k1, float('nan')) for _ in range(4)]
    want, got = grads(), grads()
    delta = torch.empty_like(lse)
    ws_bytes = lib.sa2_bwd_workspace_bytes(prob)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device='cuda')
    _native.check(lib.sa2_bwd(prob, arg(q), arg(k1), arg(k2), arg(v1), arg(v2), arg(out), arg(res), arg(dout), lse.data_ptr(),
                              saved, delta.data_ptr(), *(arg(t) for t in want), ws.data_ptr(), ws_bytes, sh))
    need = lib.sa2_bwd_noalloc_scratch_bytes(prob)
    assert 0 < need <= 64 << 20
    _native.check(lib.sa2_bwd_noalloc(prob, arg(q), arg(k1), arg(k2), arg(v1), arg(v2), arg(out), arg(res), arg(dout),
                                      lse.data_ptr(), saved, *(arg(t) for t in got), sh))
    torch.cuda.synchronize()
    for name, a, b_ in zip(U.NAMES[1:], got, want):
        assert torch.isfinite(a.float()).all(), name
        assert torch.equal(a, b_), name
    # and against the oracle, to the bar of the other parity tests
    ins = [t.cpu() for t in (q, k1, k2, v1, v2, dout)]
    ref_out, _, ref_grads = U.oracle_fwd_bwd(*ins, w1, w2)
    U.check_all(out, got, ref_out, ref_grads)


def test_no_alloc_backward_matches_the_allocating_one_twice_in_a_row():
    print('\nno-alloc backward: b=2 n=640 hq=4 hk=2 d=128 w1=200 w2=32, then b=1 n=200 hq=2 hk=2 d=64 w1=64 w2=16', flush=True)
    _backward_both_ways(2, 640, 4, 2, 128, 200, 32, seed=41, with_saved=True)
    _backward_both_ways(1, 200, 2, 2, 64, 64, 16, seed=42, with_saved=False)


def test_no_alloc_backward_refuses_what_does_not_fit():
    lib = _native.load()
    big = _native.problem(4, 8192, 8, 8, 128, 512, 32, True, 128 ** -0.5)
    assert lib.sa2_bwd_noalloc_scratch_bytes(big) > 64 << 20
    t = _native.TensorArg(0x1000, 1 << 20, 1024, 128)
    rc = lib.sa2_bwd_noalloc(big, t, t, t, t, t, t, None, t, 0x2000, None, t, t, t, t, t, None)
    assert rc == 3 and b'scratch' in lib.sa2_last_error()
