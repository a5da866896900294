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


def _pad_plan(q, v):
    """Head dims (dk, dv) to pad q / k and v to before the launch, or None.

    The flash kernels read 16-byte row pieces: head dims that are not multiples of 8 (100, 50, 36, 20, ...) would run on
    the generic kernels, 3 to 6 times slower (measured).  Zero columns appended to q, k, v (and to dO in the backward
    pass) change no score and no output column, so such calls are padded to the next multiple of 8 here and the results
    sliced back.
    """
    dk, dv = q.shape[-1], v.shape[-1]
    if q.dtype not in (torch.bfloat16, torch.float16) or max(dk, dv) > 128:
        return None
    tk, tv = (dk + 7) // 8 * 8, (dv + 7) // 8 * 8
    return None if (tk, tv) == (dk, dv) else (tk, tv)


def _pad_last(x, d):
    return x if x.shape[-1] == d else torch.nn.functional.pad(x, (0, d - x.shape[-1]))


def _cut_last(x, d):
    return x if x.shape[-1] == d else x[..., :d].contiguous()


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
        ctx.dims = (q.shape[-1], v.shape[-1])
        plan = _pad_plan(q, v)
        if plan is not None:   # head dims that are not multiples of 8: see _pad_plan
            q, k, v = _pad_last(q, plan[0]), _pad_last(k, plan[0]), _pad_last(v, plan[1])
        o, M = _forward(q, k, v, causal, sm_scale)
        ctx.save_for_backward(q, k, v, o, M)
        ctx.sm_scale = sm_scale
        ctx.causal = causal
        return _cut_last(o, ctx.dims[1])

    @staticmethod
    def backward(ctx, do):
        q, k, v, o, M = ctx.saved_tensors
        do = _pad_last(do, v.shape[-1])
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
        return _cut_last(dq, ctx.dims[0]), _cut_last(dk, ctx.dims[0]), _cut_last(dv, ctx.dims[1]), None, None


attention = _attention.apply
