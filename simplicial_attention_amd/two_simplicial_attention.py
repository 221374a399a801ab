"""Sliding-window 2-simplicial attention on MI355X: autograd Function, functional
wrapper and multi-head module.

Same names, argument order, tensor layouts and defaults as
simplicial_attention/triton_two_simplicial_attention.py of the reference
(Function :718-1008, wrapper :1020-1056, module :1062-1081); the device work is done
by hand-written gfx950 kernels reached through the C ABI of libsa2.so.
"""
from __future__ import annotations

import os
import threading
import weakref

from functools import partial

import torch
import torch.nn.functional as F
from torch import Tensor
from torch.autograd import Function

from . import _native
from .simplicial_mha import HigherOrderAttention


def _unit_inner_stride(t: Tensor) -> Tensor:
    """The kernels need a unit innermost stride, 16-byte aligned rows and base."""
    ok = (t.stride(-1) == 1 and t.data_ptr() % 16 == 0 and all(s % 8 == 0 for s in t.stride()[:-1]))
    return t if ok else t.contiguous()


def _stream_handle(device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def save_partials_max_bytes() -> int:
    """Largest per-call buffer of saved value partials the forward may allocate for the
    backward (bytes).  ``SA2_SAVE_PARTIALS_MAX_GIB`` overrides the default of 16 GiB;
    0 switches the saving off (the backward then recomputes, as the reference does)."""
    return int(float(os.environ.get('SA2_SAVE_PARTIALS_MAX_GIB', '16')) * (1 << 30))


def save_partials_total_fraction() -> float:
    """Share of a device's memory that all live saved partials together may occupy
    (``SA2_SAVE_PARTIALS_TOTAL_FRACTION``, default 0.25)."""
    return float(os.environ.get('SA2_SAVE_PARTIALS_TOTAL_FRACTION', '0.25'))


class _PartialsBudget:
    """Bytes of saved value partials alive per device (between a forward and the end of its
    backward).  The partials are ``w2`` times the size of ``q`` per call, so a deep model
    would otherwise keep ``layers * w2`` activations where the reference keeps ``layers``:
    a call saves them only while (a) the call's buffer fits the per-call cap and (b) all live
    buffers together stay below a fraction of the device's total memory.  Otherwise the
    backward recomputes, as the reference does, at about 20 % more time per layer.  The rule
    looks at sizes only, never at how much memory happens to be free: the two backward paths
    differ in the last bf16 digit of dV2, and a model's gradients must not depend on what
    else the allocator holds."""

    def __init__(self):
        self.live = {}
        self.total = {}
        self.lock = threading.Lock()

    def admit(self, nbytes: int, device, total_memory=None) -> bool:
        if nbytes <= 0 or nbytes > save_partials_max_bytes():
            return False
        index = torch.device(device).index
        index = torch.cuda.current_device() if index is None else index
        with self.lock:
            if total_memory is None:
                if index not in self.total:
                    self.total[index] = torch.cuda.get_device_properties(index).total_memory
                total_memory = self.total[index]
            live = self.live.get(index, 0)
            if live + nbytes > save_partials_total_fraction() * total_memory:
                return False
            self.live[index] = live + nbytes
        return True

    def release(self, nbytes: int, index: int) -> None:
        with self.lock:
            self.live[index] = max(self.live.get(index, 0) - nbytes, 0)

    def track(self, tensor: Tensor, nbytes: int) -> None:
        """Gives the bytes back when ``tensor`` (the saved buffer) is freed."""
        weakref.finalize(tensor, self.release, nbytes, tensor.device.index)


partials_budget = _PartialsBudget()


class SlidingTwoSimplicialAttention(Function):
    """``apply(q, k1, k2, v1, v2, w1, w2, causal[, scale]) -> out``; every tensor ``(b, n, h, d)``.

    ``k1, k2, v1, v2`` may carry fewer heads than ``q`` (grouped queries, query head
    ``h`` reads key/value head ``h // groups``); the reference's Function receives
    them already repeated, which is the special case of one group per head.
    Gradients come back in the order ``dq, dk1, dk2, dv1, dv2`` in the input dtype.
    ``scale`` (not an argument of the reference's Function, which always uses
    ``dim_head ** -0.5``) overrides the softmax scale; the functional wrapper passes it
    when it has zero-padded the head dimension.
    """

    @staticmethod
    def forward(ctx, q, k1, k2, v1, v2, w1, w2, causal, scale=None):
        tensors = (q, k1, k2, v1, v2)
        assert all(t.is_cuda for t in tensors), 'sliding-window 2-simplicial attention runs on the GPU only'
        if not causal:
            raise NotImplementedError('only causal=True is defined for the sliding windows')
        in_dtype = q.dtype
        if in_dtype not in (torch.bfloat16, torch.float16, torch.float32) or any(t.dtype != in_dtype for t in tensors):
            raise TypeError('q, k1, k2, v1, v2 must share one dtype out of bfloat16, float16, float32')
        # the kernels compute on bf16 operands with fp32 accumulation, as the reference's do for any input
        # dtype (triton_two_simplicial_attention.py:110-112, 150-152); other dtypes are cast on the way in
        # and results returned in the caller's dtype
        if in_dtype is not torch.bfloat16:
            tensors = tuple(t.to(torch.bfloat16) for t in tensors)
            q, k1, k2, v1, v2 = tensors
        if q.dim() != 4:
            raise ValueError('expected (batch, seq, heads, dim_head) tensors')
        batch, seq_len, heads, dim = q.shape
        kv_heads = k1.shape[2]
        for t in (k1, k2, v1, v2):
            if t.shape != (batch, seq_len, kv_heads, dim):
                raise ValueError(f'key/value shape {tuple(t.shape)} does not match {(batch, seq_len, kv_heads, dim)}')
        if heads % kv_heads != 0:
            raise ValueError(f'query heads {heads} not divisible by key/value heads {kv_heads}')
        w1, w2 = int(w1), int(w2)
        if w1 < 1 or w2 < 1:
            raise ValueError('window sizes must be at least 1')
        lib = _native.load()
        if not lib.sa2_supported(dim, w1, w2, _native.SA2_BF16):
            raise NotImplementedError(f'dim_head={dim}, w1={w1}, w2={w2} is not covered by the kernels (dim_head 32, 64, 128 or 256)')

        q, k1, k2, v1, v2 = (_unit_inner_stride(t) for t in tensors)
        scale = dim ** -0.5 if scale is None else float(scale)
        out = torch.empty((batch, seq_len, heads, dim), dtype=q.dtype, device=q.device)
        lse = torch.empty((batch, heads, seq_len), dtype=torch.float32, device=q.device)
        # bf16 residual of the fp32 accumulator, kept only when a backward may follow
        needs_grad = any(ctx.needs_input_grad[:5])
        residual = torch.empty_like(out) if needs_grad else None
        prob = _native.problem(batch, seq_len, heads, kv_heads, dim, w1, w2, True, scale)
        # per-offset value partials T (and their references), kept for the backward when
        # they fit the budget: dV2 then needs no recomputation of the attention weights
        t_save = m_save = None
        t_bytes = lib.sa2_saved_t_bytes(prob) + lib.sa2_saved_m_bytes(prob)
        # (a size of 0: this head dimension's kernels keep no partials)
        if needs_grad and t_bytes > 0 and partials_budget.admit(t_bytes, q.device):
            try:
                t_save = torch.empty(lib.sa2_saved_t_bytes(prob), dtype=torch.uint8, device=q.device)
                m_save = torch.empty((batch, heads, w2, seq_len), dtype=torch.float32, device=q.device)
            except BaseException:
                # (no buffer to hang the release on: give the admitted bytes back here)
                index = q.device.index if q.device.index is not None else torch.cuda.current_device()
                partials_budget.release(t_bytes, index)
                raise
            partials_budget.track(t_save, t_bytes)
        with torch.cuda.device_of(q):
            _native.check(lib.sa2_fwd(prob, *(_native.tensor_arg(t) for t in (q, k1, k2, v1, v2, out)),
                                      _native.tensor_arg(residual) if needs_grad else None,
                                      lse.data_ptr(),
                                      _native.saved_arg(t_save, m_save) if t_save is not None else None,
                                      _stream_handle(q.device)))
        ctx.save_for_backward(q, k1, k2, v1, v2, out, lse, residual, t_save, m_save)
        ctx.problem = (batch, seq_len, heads, kv_heads, dim, w1, w2, scale)
        ctx.in_dtype = in_dtype
        return out if in_dtype is torch.bfloat16 else out.to(in_dtype)

    @staticmethod
    def backward(ctx, dout):
        q, k1, k2, v1, v2, out, lse, residual, t_save, m_save = ctx.saved_tensors
        batch, seq_len, heads, kv_heads, dim, w1, w2, scale = ctx.problem
        dout = _unit_inner_stride(dout if dout.dtype is torch.bfloat16 else dout.to(torch.bfloat16))
        lib = _native.load()
        delta = torch.empty_like(lse)
        dq = torch.empty_like(q)
        dk1, dk2, dv1, dv2 = (torch.empty((batch, seq_len, kv_heads, dim), dtype=q.dtype, device=q.device) for _ in range(4))
        prob = _native.problem(batch, seq_len, heads, kv_heads, dim, w1, w2, True, scale)
        # (with the forward's saved partials only the dK2 half of the workspace is used)
        ws_bytes = lib.sa2_bwd_workspace_bytes_with_saved(prob) if t_save is not None else lib.sa2_bwd_workspace_bytes(prob)
        workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device)
        arg = _native.tensor_arg
        with torch.cuda.device_of(q):
            _native.check(lib.sa2_bwd(prob, arg(q), arg(k1), arg(k2), arg(v1), arg(v2), arg(out),
                                      arg(residual) if residual is not None else None, arg(dout),
                                      lse.data_ptr(),
                                      _native.saved_arg(t_save, m_save) if t_save is not None else None,
                                      delta.data_ptr(),
                                      arg(dq), arg(dk1), arg(dk2), arg(dv1), arg(dv2),
                                      workspace.data_ptr(), ws_bytes, _stream_handle(q.device)))
        if ctx.in_dtype is not torch.bfloat16:
            dq, dk1, dk2, dv1, dv2 = (t.to(ctx.in_dtype) for t in (dq, dk1, dk2, dv1, dv2))
        return dq, dk1, dk2, dv1, dv2, None, None, None, None


_sliding_two_simplicial_attn = SlidingTwoSimplicialAttention.apply


def sliding_two_simplicial_attn(
    q: Tensor,                      # (b, n, hq, d)
    keys: tuple[Tensor, Tensor],    # (b, n, h, d) * 2
    values: tuple[Tensor, Tensor],  # (b, n, h, d) * 2
    w1=512,
    w2=32,
    causal=True,
    pad_to_multiple_of=64,
):
    """Functional entry point, signature of triton_two_simplicial_attention.py:1020-1056.

    Grouped-query heads are resolved by index arithmetic inside the kernels and a
    ragged sequence end is masked there, so nothing is repeated or padded here;
    ``pad_to_multiple_of`` is accepted for compatibility and has no effect on the
    result (zero rows appended after a causal sequence cannot influence it).

    Beyond the reference (whose kernels are written for bf16 and a head dimension of
    64): float16 and float32 tensors are computed in bfloat16 and the result returned
    in the input dtype; any head dimension up to 256, and a value head dimension
    different from the query/key one, are zero-padded to the kernels' 32, 64, 128 or 256
    (padded query/key channels add nothing to the logits, padded value channels give
    zero outputs that are sliced off; the softmax scale stays that of the true
    query/key dimension).
    """
    if len(keys) != 2 or len(values) != 2:
        raise AssertionError('two key sets and two value sets are required')
    q_heads, k_heads = q.shape[-2], keys[0].shape[-2]
    assert q_heads % k_heads == 0, 'query heads must be a multiple of key/value heads'
    (k1, k2), (v1, v2) = keys, values
    dtype, dim_qk, dim_v = q.dtype, q.shape[-1], v1.shape[-1]
    if dtype not in (torch.bfloat16, torch.float16, torch.float32):
        raise TypeError(f'unsupported dtype {dtype}')
    if k1.shape[-1] != dim_qk or k2.shape[-1] != dim_qk or v2.shape[-1] != dim_v:
        raise ValueError('q, k1, k2 must share one head dimension and v1, v2 another')
    dim = max(dim_qk, dim_v)
    if dim > 256:
        raise NotImplementedError(f'head dimension {dim} is not covered by the kernels (at most 256)')
    if dtype is torch.bfloat16 and dim_qk == dim_v and dim in (32, 64, 128, 256):
        return _sliding_two_simplicial_attn(q, k1, k2, v1, v2, w1, w2, causal)
    dim_kernel = next(d for d in (32, 64, 128, 256) if dim <= d)

    def prepare(t):
        t = t.to(torch.bfloat16)
        return F.pad(t, (0, dim_kernel - t.shape[-1])) if t.shape[-1] != dim_kernel else t

    out = _sliding_two_simplicial_attn(*(prepare(t) for t in (q, k1, k2, v1, v2)), w1, w2, causal, dim_qk ** -0.5)
    return out[..., :dim_v].to(dtype)


class SlidingWindowTwoSimplicialMHA(HigherOrderAttention):
    """Multi-head module, constructor of triton_two_simplicial_attention.py:1062-1081."""

    def __init__(self, *args, w1=512, w2=32, **kwargs):
        assert 'number_key_value_sets' not in kwargs
        assert 'head_first_dim' not in kwargs
        attend = partial(sliding_two_simplicial_attn, w1=w1, w2=w2, causal=True)
        super().__init__(*args, number_key_value_sets=2, head_first_dim=False, attend=attend, **kwargs)
