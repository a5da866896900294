"""Tiled 2D sliding-window flash attention (drop-in for src/tiled_swa.py).

``TiledSwa`` keeps the reference's autograd contract (src/tiled_swa.py:602-689): positional
arguments ``(q, k, v, b_size, t_height, t_width, row_size, col_size, sm_scale)`` and a
backward that returns ``(dq, dk, dv, None * 6)``.  ``tiled_swa_fwd`` (:564-600) is the no-grad
forward.  Deliberate differences from the reference, all documented in the C header:
outputs have the dtype and device of ``q`` (the reference hard-codes fp16 and the default
device, :608-609), the saved log-sum-exp is fp32, and tiles smaller than 16 tokens have a
backward (the reference raises, :660-661).

``TiledSwaRope`` is the fused RoPE-2D + attention op: it equals ``RotaryPE2D`` applied to
q and k followed by ``TiledSwa`` (the composition of README.md:11) with the caller's q and k
left untouched; its backward returns gradients for the un-rotated q and k.

``TiledSwaImage`` takes q, k, v as images ``[B, IH, IW, heads, D]`` (the layout the reference's
demo converts from with reshape / permute / reshape, src/tiled_swa.py:753-755) and returns o in
the same layout; the kernels address pixels themselves, so no permuted copy is made on either side.
"""
from __future__ import annotations

import torch

from . import _lib


def _shape(q, k, v, b_size, t_height, t_width, row_size, col_size, sm_scale) -> _lib.SwaShape:
    B, H, N, KEY_DIM = q.shape
    HEAD_DIM = v.shape[-1]
    assert N == t_height * t_width * b_size, "seqlen should match image size"
    assert k.shape == (B, H, N, KEY_DIM) and v.shape[:3] == (B, H, N)
    assert q.dtype == k.dtype == v.dtype
    return _lib.SwaShape(B, H, b_size, t_height, t_width, row_size, col_size, KEY_DIM, HEAD_DIM, float(sm_scale),
                         _lib.dtype_code(q))


def _pad_plan(q, v, b_size):
    """Head dims (dk, dv) to pad q / k and v to before the launch, or None.

    The tuned token-grid kernels (``b_size == 1``) take head dims that are multiples of 32 with both in one class (both
    <= 64, or both in 65..128); anything else runs on the generic kernels, 6 to 9 times slower (measured at d = 40, 48,
    80 against 64, 96, 128).  Zero columns appended to q, k, v (and to dO in the backward pass) change no score and no
    output column, so such calls are padded to the next tuned shape here and the results sliced back: four to eight
    extra copy passes over the tensors, a few percent of the step.  Tiles of 16 k tokens need none of this: their
    kernels pad inside.
    """
    dk, dv = q.shape[-1], v.shape[-1]
    if q.dtype not in (torch.bfloat16, torch.float16) or max(dk, dv) > 128:
        return None
    if 2 <= b_size <= 15:
        # tiles of fewer than 16 tokens run on the streaming token-grid kernels at head dim 64 or 128 exactly (both equal);
        # the generic kernels they would use otherwise are 2 to 4 times slower
        t = 64 if max(dk, dv) <= 64 else 128
        return None if (dk, dv) == (t, t) else (t, t)
    if b_size != 1:
        return None
    up = lambda d: (d + 31) // 32 * 32
    tk, tv = (up(dk), up(dv)) if max(dk, dv) <= 64 else (max(96, up(dk)), max(96, up(dv)))
    return None if (tk, tv) == (dk, dv) else (tk, tv)


def _pad_last(x, d):
    return x if x.shape[-1] == d else torch.nn.functional.pad(x, (0, d - x.shape[-1]))


def _cut_last(x, d):
    return x if x.shape[-1] == d else x[..., :d].contiguous()


def _forward(q, k, v, shape, rope):
    _lib.require_cuda(q, k, v)
    lib = _lib.load()
    B, H, N, _ = q.shape
    o = torch.empty((B, H, N, v.shape[-1]), dtype=q.dtype, device=q.device)
    lse = torch.empty((B, H, N), dtype=torch.float32, device=q.device)
    desc, keep = (None, None) if rope is None else _lib.rope_desc(*rope, like=q, n_tokens=q.shape[2])
    with torch.cuda.device(q.device):
        _lib.check(lib.dlt_swa_fwd(_lib.ptr(q), _lib.strides(q), _lib.ptr(k), _lib.strides(k), _lib.ptr(v),
                                   _lib.strides(v), _lib.ptr(o), _lib.strides(o), _lib.ptr(lse), _lib.strides(lse),
                                   shape, desc, _lib.stream_of(q)))
    del keep
    return o, lse


def _backward(q, k, v, o, lse, do, shape, rope):
    lib = _lib.load()
    _lib.require_cuda(q, k, v, o, lse, do)
    dq = torch.empty_like(q)
    dk = torch.empty_like(k)
    dv = torch.empty_like(v)
    delta = torch.empty_like(lse)
    desc, keep = (None, None) if rope is None else _lib.rope_desc(*rope, like=q, n_tokens=q.shape[2])
    with torch.cuda.device(q.device):
        _lib.check(lib.dlt_swa_bwd(_lib.ptr(q), _lib.strides(q), _lib.ptr(k), _lib.strides(k), _lib.ptr(v),
                                   _lib.strides(v), _lib.ptr(o), _lib.strides(o), _lib.ptr(do), _lib.strides(do),
                                   _lib.ptr(lse), _lib.ptr(delta), _lib.strides(lse),
                                   _lib.ptr(dq), _lib.strides(dq), _lib.ptr(dk), _lib.strides(dk),
                                   _lib.ptr(dv), _lib.strides(dv), shape, desc, _lib.stream_of(q)))
    del keep
    return dq, dk, dv


def tiled_swa_fwd(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, b_size: int, t_height: int, t_width: int,
                  row_size: int, col_size: int, sm_scale: float = 1.0):
    dv, plan = v.shape[-1], _pad_plan(q, v, b_size)
    if plan is not None:
        q, k, v = _pad_last(q, plan[0]), _pad_last(k, plan[0]), _pad_last(v, plan[1])
    shape = _shape(q, k, v, b_size, t_height, t_width, row_size, col_size, sm_scale)
    return _cut_last(_forward(q, k, v, shape, None)[0], dv)


class TiledSwa(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, b_size: int, t_height: int, t_width: int,
                row_size: int, col_size: int, sm_scale: float):
        ctx.dims = (q.shape[-1], v.shape[-1])
        plan = _pad_plan(q, v, b_size)
        if plan is not None:   # head dims outside the tuned token-grid shapes: see _pad_plan
            q, k, v = _pad_last(q, plan[0]), _pad_last(k, plan[0]), _pad_last(v, plan[1])
        shape = _shape(q, k, v, b_size, t_height, t_width, row_size, col_size, sm_scale)
        o, m = _forward(q, k, v, shape, None)
        ctx.save_for_backward(q, k, v, m, o)
        o = _cut_last(o, ctx.dims[1])
        ctx.b_size = b_size
        ctx.t_height = t_height
        ctx.t_width = t_width
        ctx.row_size = row_size
        ctx.col_size = col_size
        ctx.sm_scale = sm_scale
        return o

    @staticmethod
    def backward(ctx, do: torch.Tensor):
        q, k, v, m, o = ctx.saved_tensors
        shape = _shape(q, k, v, ctx.b_size, ctx.t_height, ctx.t_width, ctx.row_size, ctx.col_size, ctx.sm_scale)
        dq, dk, dv = _backward(q, k, v, o, m, _pad_last(do, v.shape[-1]), shape, None)
        dq, dk, dv = _cut_last(dq, ctx.dims[0]), _cut_last(dk, ctx.dims[0]), _cut_last(dv, ctx.dims[1])
        return dq, dk, dv, None, None, None, None, None, None,


def _forward_rot(q, k, v, shape, rope):
    """Forward of the fused op that also returns the rotated q and k (kept for the backward pass)."""
    _lib.require_cuda(q, k, v)
    B, H, N, _ = q.shape
    o = torch.empty((B, H, N, v.shape[-1]), dtype=q.dtype, device=q.device)
    lse = torch.empty((B, H, N), dtype=torch.float32, device=q.device)
    desc, keep = _lib.rope_desc(*rope, like=q, n_tokens=q.shape[2])
    q_rot = torch.empty(q.shape, dtype=q.dtype, device=q.device)
    k_rot = torch.empty(k.shape, dtype=k.dtype, device=k.device)
    with torch.cuda.device(q.device):
        _lib.check(_lib.load().dlt_swa_fwd_rot(
            _lib.ptr(q), _lib.strides(q), _lib.ptr(k), _lib.strides(k), _lib.ptr(v), _lib.strides(v),
            _lib.ptr(o), _lib.strides(o), _lib.ptr(lse), _lib.strides(lse),
            _lib.ptr(q_rot), _lib.strides(q_rot), _lib.ptr(k_rot), _lib.strides(k_rot), shape, desc, _lib.stream_of(q)))
    del keep
    return o, lse, q_rot, k_rot


def _backward_rot(q_rot, k_rot, v, o, lse, do, shape, rope):
    _lib.require_cuda(q_rot, k_rot, v, o, lse, do)
    dq, dk, dv = torch.empty_like(q_rot), torch.empty_like(k_rot), torch.empty_like(v)
    delta = torch.empty_like(lse)
    desc, keep = _lib.rope_desc(*rope, like=v, n_tokens=v.shape[2])
    with torch.cuda.device(v.device):
        _lib.check(_lib.load().dlt_swa_bwd_rot(
            _lib.ptr(q_rot), _lib.strides(q_rot), _lib.ptr(k_rot), _lib.strides(k_rot), _lib.ptr(v), _lib.strides(v),
            _lib.ptr(o), _lib.strides(o), _lib.ptr(do), _lib.strides(do),
            _lib.ptr(lse), _lib.ptr(delta), _lib.strides(lse),
            _lib.ptr(dq), _lib.strides(dq), _lib.ptr(dk), _lib.strides(dk), _lib.ptr(dv), _lib.strides(dv),
            shape, desc, _lib.stream_of(v)))
    del keep
    return dq, dk, dv


class TiledSwaRope(torch.autograd.Function):
    """o = TiledSwa(rope(q), rope(k), v) with the rotation fused into the q / k tile loads.

    ``save_rotated`` (optional last argument of ``apply``, default True): the forward pass also stores the
    rotated q and k (what ``RotaryPE2D`` leaves in place in the reference's composition) and the backward pass
    reads those, rotating only dq and dk back as they are stored.  False keeps nothing but the caller's q and k
    and rotates every staged tile again in the backward kernels: two tensors less memory, slower.  It is a
    per-call argument, kept in the call's own context: nothing is shared between calls or threads.
    """

    @staticmethod
    def forward(ctx, q, k, v, idx, row_cs_buffer, col_cs_buffer, b_size, t_height, t_width, row_size, col_size,
                sm_scale, save_rotated=None):
        ctx.n_inputs = 12 if save_rotated is None else 13   # backward returns one entry per argument of apply
        ctx.dims = (q.shape[-1], v.shape[-1])
        plan = _pad_plan(q, v, b_size)
        if plan is not None:   # zero columns behind the rotated ones: see _pad_plan
            q, k, v = _pad_last(q, plan[0]), _pad_last(k, plan[0]), _pad_last(v, plan[1])
        shape = _shape(q, k, v, b_size, t_height, t_width, row_size, col_size, sm_scale)
        assert row_cs_buffer.shape[1] == col_cs_buffer.shape[1]
        assert idx.shape[0] == q.shape[2]
        rope = (idx, row_cs_buffer, col_cs_buffer)
        ctx.rotated = True if save_rotated is None else bool(save_rotated)
        if ctx.rotated:
            o, m, q_rot, k_rot = _forward_rot(q, k, v, shape, rope)
            ctx.save_for_backward(q_rot, k_rot, v, m, o, idx, row_cs_buffer, col_cs_buffer)
        else:
            o, m = _forward(q, k, v, shape, rope)
            ctx.save_for_backward(q, k, v, m, o, idx, row_cs_buffer, col_cs_buffer)
        ctx.scalars = (b_size, t_height, t_width, row_size, col_size, sm_scale)
        return _cut_last(o, ctx.dims[1])

    @staticmethod
    def backward(ctx, do):
        q, k, v, m, o, idx, row_cs_buffer, col_cs_buffer = ctx.saved_tensors
        shape = _shape(q, k, v, *ctx.scalars)
        rope = (idx, row_cs_buffer, col_cs_buffer)
        do = _pad_last(do, v.shape[-1])
        if ctx.rotated:
            dq, dk, dv = _backward_rot(q, k, v, o, m, do, shape, rope)
        else:
            dq, dk, dv = _backward(q, k, v, o, m, do, shape, rope)
        dq, dk, dv = _cut_last(dq, ctx.dims[0]), _cut_last(dk, ctx.dims[0]), _cut_last(dv, ctx.dims[1])
        return (dq, dk, dv) + (None,) * (ctx.n_inputs - 3)


def _image_shape(q, k, v, bh, bw, row_size, col_size, sm_scale):
    B, IH, IW, H, KEY_DIM = q.shape
    assert IH % bh == 0 and IW % bw == 0, "image size should be a multiple of the tile size"
    assert k.shape == q.shape and v.shape[:4] == q.shape[:4]
    assert q.dtype == k.dtype == v.dtype
    shape = _lib.SwaShape(B, H, bh * bw, IH // bh, IW // bw, row_size, col_size, KEY_DIM, v.shape[-1], float(sm_scale),
                          _lib.dtype_code(q))
    return shape, _lib.SwaTile(bh, bw)


class TiledSwaImage(torch.autograd.Function):
    """``TiledSwa`` on image-layout tensors: q, k ``[B, IH, IW, heads, dk]``, v and o ``[B, IH, IW, heads, dv]``.

    A tile is a block of ``bh x bw`` pixels (``b_size = bh * bw``); the window is ``row_size`` / ``col_size``
    tiles to each side as in ``TiledSwa``.  Equals the reference's conversion to ``[B, heads, N, D]``
    (src/tiled_swa.py:753-755, inverted), ``TiledSwa`` and the conversion back, without the copies.
    """

    @staticmethod
    def forward(ctx, q, k, v, bh: int, bw: int, row_size: int, col_size: int, sm_scale: float):
        shape, tile = _image_shape(q, k, v, bh, bw, row_size, col_size, sm_scale)
        _lib.require_cuda(q, k, v)
        B, IH, IW, H, _ = q.shape
        o = torch.empty((B, IH, IW, H, v.shape[-1]), dtype=q.dtype, device=q.device)
        lse = torch.empty((B, H, IH * IW), dtype=torch.float32, device=q.device)
        with torch.cuda.device(q.device):
            _lib.check(_lib.load().dlt_swa_fwd_image(
                _lib.ptr(q), _lib.strides(q), _lib.ptr(k), _lib.strides(k), _lib.ptr(v), _lib.strides(v),
                _lib.ptr(o), _lib.strides(o), _lib.ptr(lse), _lib.strides(lse), shape, tile, None, _lib.stream_of(q)))
        ctx.save_for_backward(q, k, v, lse, o)
        ctx.scalars = (bh, bw, row_size, col_size, sm_scale)
        return o

    @staticmethod
    def backward(ctx, do):
        q, k, v, lse, o = ctx.saved_tensors
        shape, tile = _image_shape(q, k, v, *ctx.scalars)
        _lib.require_cuda(q, k, v, o, lse, do)
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        delta = torch.empty_like(lse)
        with torch.cuda.device(q.device):
            _lib.check(_lib.load().dlt_swa_bwd_image(
                _lib.ptr(q), _lib.strides(q), _lib.ptr(k), _lib.strides(k), _lib.ptr(v), _lib.strides(v),
                _lib.ptr(o), _lib.strides(o), _lib.ptr(do), _lib.strides(do),
                _lib.ptr(lse), _lib.ptr(delta), _lib.strides(lse),
                _lib.ptr(dq), _lib.strides(dq), _lib.ptr(dk), _lib.strides(dk), _lib.ptr(dv), _lib.strides(dv),
                shape, tile, None, _lib.stream_of(q)))
        return (dq, dk, dv) + (None,) * 5


def swa_image_offsets(t_height: int, t_width: int, bh: int, bw: int, stride_y: int, stride_x: int,
                      device="cuda") -> torch.Tensor:
    """int64 [N]: element offset of every token's pixel, computed by the kernels' own token -> pixel routine."""
    out = torch.empty((t_height * t_width * bh * bw,), dtype=torch.int64, device=device)
    with torch.cuda.device(out.device):
        _lib.check(_lib.load().dlt_swa_image_offsets(t_height, t_width, bh, bw, stride_y, stride_x, _lib.ptr(out),
                                                     _lib.stream_of(out)))
    return out


def swa_neighbors(t_height: int, t_width: int, row_size: int, col_size: int, device="cuda") -> torch.Tensor:
    """bool [T, T] neighbour mask computed on the device by the kernels' own window routine."""
    T = t_height * t_width
    out = torch.empty((T, T), dtype=torch.uint8, device=device)
    with torch.cuda.device(out.device):
        _lib.check(_lib.load().dlt_swa_neighbors(t_height, t_width, row_size, col_size, _lib.ptr(out),
                                                 _lib.stream_of(out)))
    return out.bool()
