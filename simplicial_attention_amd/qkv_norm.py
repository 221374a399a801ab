"""Fused split + per-head RMSNorm of the qkv projection (autograd Function over libsa2).

Does in one kernel what HigherOrderAttention.forward does between the ``to_qkv``
projection and the attention call when there are two key/value sets and heads are not
moved in front of the sequence (simplicial_mha.py:116-127 of the reference): split into
q | k | v, unflatten heads with channel order ``(head, set, d)``, chunk the sets apart and
apply the five ``RMSNorm(dim_head)`` modules.
"""
from __future__ import annotations

import torch
from torch.autograd import Function

from . import _native


def _ptr(t):
    return None if t is None else t.data_ptr()


class FusedQKVNorm(Function):
    """``apply(qkv, wq, wk1, wk2, wv1, wv2, heads, kv_heads, dim_head, eps) -> q, k1, k2, v1, v2``.

    ``qkv``: (b, n, (heads + 4 kv_heads) * dim_head) bf16 on the GPU; the weights are the
    ``weight`` tensors of the five RMSNorm modules (bf16, ``(dim_head,)``) or ``None``.
    Outputs are contiguous (b, n, h, dim_head).
    """

    @staticmethod
    def forward(ctx, qkv, wq, wk1, wk2, wv1, wv2, heads, kv_heads, dim_head, eps):
        assert qkv.is_cuda and qkv.dtype == torch.bfloat16 and qkv.dim() == 3
        batch, seq_len, channels = qkv.shape
        assert channels == (heads + 4 * kv_heads) * dim_head, 'projection width does not match the head layout'
        qkv = qkv if qkv.stride(-1) == 1 and qkv.stride(0) == seq_len * qkv.stride(1) else qkv.contiguous()
        weights = [None if w is None else w.detach().to(torch.bfloat16).contiguous() for w in (wq, wk1, wk2, wv1, wv2)]
        lib = _native.load()
        prob = _native.problem(batch, seq_len, heads, kv_heads, dim_head, 1, 1, True, 1.0)
        mk = lambda h: torch.empty((batch, seq_len, h, dim_head), dtype=qkv.dtype, device=qkv.device)
        outs = [mk(heads)] + [mk(kv_heads) for _ in range(4)]
        rstd = torch.empty((batch * seq_len, heads + 4 * kv_heads), dtype=torch.float32, device=qkv.device)
        with torch.cuda.device_of(qkv):
            _native.check(lib.sa2_qkv_norm_fwd(prob, qkv.data_ptr(), qkv.stride(1), *(_ptr(w) for w in weights), float(eps),
                                               *(_native.tensor_arg(t) for t in outs), rstd.data_ptr(),
                                               torch.cuda.current_stream(qkv.device).cuda_stream))
        ctx.save_for_backward(qkv, rstd, *[w for w in weights if w is not None])
        ctx.has_weight = [w is not None for w in weights]
        ctx.weight_dtypes = [None if w is None else w.dtype for w in (wq, wk1, wk2, wv1, wv2)]
        ctx.geometry = (batch, seq_len, heads, kv_heads, dim_head)
        return tuple(outs)

    @staticmethod
    def backward(ctx, dq, dk1, dk2, dv1, dv2):
        qkv, rstd, *present = ctx.saved_tensors
        it = iter(present)
        weights = [next(it) if has else None for has in ctx.has_weight]
        batch, seq_len, heads, kv_heads, dim_head = ctx.geometry
        lib = _native.load()
        prob = _native.problem(batch, seq_len, heads, kv_heads, dim_head, 1, 1, True, 1.0)
        grads = [g.contiguous() for g in (dq, dk1, dk2, dv1, dv2)]
        dqkv = torch.empty((batch, seq_len, qkv.shape[-1]), dtype=qkv.dtype, device=qkv.device)
        dw = torch.empty((5, dim_head), dtype=torch.float32, device=qkv.device)
        ws_bytes = lib.sa2_qkv_norm_bwd_workspace_bytes(prob)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=qkv.device)
        with torch.cuda.device_of(qkv):
            _native.check(lib.sa2_qkv_norm_bwd(prob, qkv.data_ptr(), qkv.stride(1), *(_ptr(w) for w in weights),
                                               *(_native.tensor_arg(g) for g in grads), rstd.data_ptr(), dqkv.data_ptr(),
                                               dw.data_ptr(), ws.data_ptr(), ws_bytes,
                                               torch.cuda.current_stream(qkv.device).cuda_stream))
        dws = [dw[x].to(dt) if has else None for x, (has, dt) in enumerate(zip(ctx.has_weight, ctx.weight_dtypes))]
        return (dqkv, *dws, None, None, None, None)


def fused_qkv_norm(qkv, norms, heads, kv_heads, dim_head):
    """``norms``: the five RMSNorm modules in the order q, k1, k2, v1, v2."""
    # eps=None: torch's rms_norm normalises bf16 input in fp32 with the fp32 machine epsilon
    eps = norms[0].eps if norms[0].eps is not None else torch.finfo(torch.float32).eps
    weights = [n.weight if n.elementwise_affine else None for n in norms]
    return FusedQKVNorm.apply(qkv, *weights, heads, kv_heads, dim_head, eps)
