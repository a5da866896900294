"""Flash attention with separate qk / vo head dims (drop-in for src/flash_attn.py).

``attention(q, k, v, causal, sm_scale)`` = ``_attention.apply`` as in the reference
(src/flash_attn.py:452-541); backward returns ``(dq, dk, dv, None, None)``.  Unlike the
reference (one N_CTX, :479) the key length may differ from the query length when
``causal`` is False, and there is no ``N_CTX % 128`` requirement (:512).
"""
from __future__ import annotations

import torch

from . import _lib


def _shape(q, k, v, causal, sm_scale) -> _lib.FlashShape:
    HEAD_DIM_Q, HEAD_DIM_K = q.shape[-1], k.shape[-1]
    HEAD_DIM_V = v.shape[-1]
    assert HEAD_DIM_Q == HEAD_DIM_K
    assert q.shape[:2] == k.shape[:2] == v.shape[:2] and k.shape[2] == v.shape[2]
    assert q.dtype == k.dtype == v.dtype
    return _lib.FlashShape(q.shape[0], q.shape[1], q.shape[2], k.shape[2], HEAD_DIM_K, HEAD_DIM_V, float(sm_scale),
                           int(bool(causal)), _lib.dtype_code(q))


def _forward(q, k, v, causal, sm_scale):
    """(o, M): the output and the saved log2-domain log-sum-exp [B, H, Lq] (src/flash_attn.py:463-483)."""
    shape = _shape(q, k, v, causal, sm_scale)
    _lib.require_cuda(q, k, v)
    lib = _lib.load()
    o = torch.empty((q.shape[0], q.shape[1], q.shape[2], v.shape[-1]), dtype=q.dtype, device=q.device)
    M = torch.empty((q.shape[0], q.shape[1], q.shape[2]), device=q.device, dtype=torch.float32)
    with torch.cuda.device(q.device):
        _lib.check(lib.dlt_flash_fwd(_lib.ptr(q), _lib.strides(q), _lib.ptr(k), _lib.strides(k), _lib.ptr(v),
                                     _lib.strides(v), _lib.ptr(o), _lib.strides(o), _lib.ptr(M), _lib.strides(M),
                                     shape, _lib.stream_of(q)))
    return o, M


class _attention(torch.autograd.Function):

    @staticmethod
    def forward(ctx, q, k, v, causal, sm_scale):
        o, M = _forward(q, k, v, causal, sm_scale)
        ctx.save_for_backward(q, k, v, o, M)
        ctx.sm_scale = sm_scale
        ctx.causal = causal
        return o

    @staticmethod
    def backward(ctx, do):
        q, k, v, o, M = ctx.saved_tensors
        shape = _shape(q, k, v, ctx.causal, ctx.sm_scale)
        lib = _lib.load()
        dq = torch.empty_like(q)
        dk = torch.empty_like(k)
        dv = torch.empty_like(v)
        delta = torch.empty_like(M)
        with torch.cuda.device(q.device):
            _lib.check(lib.dlt_flash_bwd(_lib.ptr(q), _lib.strides(q), _lib.ptr(k), _lib.strides(k), _lib.ptr(v),
                                         _lib.strides(v), _lib.ptr(o), _lib.strides(o), _lib.ptr(do), _lib.strides(do),
                                         _lib.ptr(M), _lib.ptr(delta), _lib.strides(M),
                                         _lib.ptr(dq), _lib.strides(dq), _lib.ptr(dk), _lib.strides(dk),
                                         _lib.ptr(dv), _lib.strides(dv), shape, _lib.stream_of(q)))
        return dq, dk, dv, None, None


attention = _attention.apply
