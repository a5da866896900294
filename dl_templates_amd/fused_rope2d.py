"""Fused in-place 2D rotary position encoding (drop-in for src/fused_rope2d.py).

Same names and call signatures as the reference: ``RotaryPE2D`` (autograd.Function,
src/fused_rope2d.py:124-168), ``FusedInplaceRotaryPositionEncoding2D`` (:171-201).  The
Triton kernels are replaced by the gfx950 HIP kernel behind ``dlt_rope2d``.
"""
from __future__ import annotations

import torch

from . import _lib
from .rope2d import FusedRotaryPositionEncodingContext


def _launch(x: torch.Tensor, idx, row_cs, col_cs, inverse: bool) -> None:
    _lib.require_cuda(x, idx, row_cs, col_cs)
    lib = _lib.load()
    desc, keep = _lib.rope_desc(idx, row_cs, col_cs)
    B, N, C = x.shape
    with torch.cuda.device(x.device):
        _lib.check(lib.dlt_rope2d(_lib.ptr(x), _lib.strides(x), B, N, C, desc, int(inverse),
                                  _lib.dtype_code(x), _lib.stream_of(x)))
    del keep


class RotaryPE2D(torch.autograd.Function):
    """x[B', N, C] is rotated IN PLACE and returned (src/fused_rope2d.py:126-145)."""

    @staticmethod
    def forward(ctx, x: torch.Tensor, idx: torch.Tensor, row_cs_buffer: torch.Tensor, col_cs_buffer: torch.Tensor):
        B, N, N_DIM = x.shape
        assert row_cs_buffer.shape[1] == col_cs_buffer.shape[1]
        assert idx.shape[0] == N
        _launch(x, idx, row_cs_buffer, col_cs_buffer, inverse=False)
        ctx.mark_dirty(x)
        ctx.save_for_backward(idx, row_cs_buffer, col_cs_buffer)
        return x

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, do: torch.Tensor):
        idx, row_cs_buffer, col_cs_buffer = ctx.saved_tensors
        dx = do.clone()
        B, N, N_DIM = dx.shape
        assert row_cs_buffer.shape[1] == col_cs_buffer.shape[1]
        assert idx.shape[0] == N
        _launch(dx, idx, row_cs_buffer, col_cs_buffer, inverse=True)
        return dx, None, None, None


def rope2d_qk_(q: torch.Tensor, k: torch.Tensor, idx: torch.Tensor, row_cs_buffer: torch.Tensor,
               col_cs_buffer: torch.Tensor, inverse: bool = False):
    """Rotate q[B, H, N, C] and k[B, H, N, C] in place with ONE launch (no autograd).

    Equivalent to two ``RotaryPE2D`` forward calls; halves the launch count and shares the
    idx / table reads (the composition of README.md:11)."""
    _lib.require_cuda(q, k, idx, row_cs_buffer, col_cs_buffer)
    assert q.shape[-2:] == k.shape[-2:] and q.dtype == k.dtype
    N, C = q.shape[-2:]
    q3, k3 = q.view(-1, N, C), k.view(-1, N, C)
    lib = _lib.load()
    desc, keep = _lib.rope_desc(idx, row_cs_buffer, col_cs_buffer)
    with torch.cuda.device(q.device):
        _lib.check(lib.dlt_rope2d_pair(_lib.ptr(q3), _lib.strides(q3), q3.shape[0], _lib.ptr(k3), _lib.strides(k3),
                                       k3.shape[0], N, C, desc, int(inverse), _lib.dtype_code(q), _lib.stream_of(q)))
    del keep
    return q, k


def rope_pe_mask(idx: torch.Tensor) -> torch.Tensor:
    """uint8[N]: bit0 = row axis rotated, bit1 = column axis rotated, decoded on the device by
    the code the rotation kernels use (src/fused_rope2d.py:40-45)."""
    _lib.require_cuda(idx)
    out = torch.empty(idx.shape[0], dtype=torch.uint8, device=idx.device)
    with torch.cuda.device(idx.device):
        _lib.check(_lib.load().dlt_rope_pe_mask(_lib.ptr(idx), idx.shape[0], _lib.ptr(out), _lib.stream_of(idx)))
    return out


class FusedInplaceRotaryPositionEncoding2D(torch.nn.Module):
    @staticmethod
    def encode_idx(height: int, width: int) -> torch.Tensor:
        r"""Token indices for image-like 2D data: ``(row << 16) | col``, row-major, int32
        (src/fused_rope2d.py:173-183)."""
        rows = torch.arange(0, height)
        cols = torch.arange(0, width)
        return torch.bitwise_or(rows[:, None] << 16, cols).flatten().to(torch.int32)

    def __init__(self, n_components: int, max_h: int, max_w: int):
        super().__init__()
        self.max_h = max_h
        self.max_w = max_w
        self.row_components = n_components // 2
        self.col_components = n_components // 2
        self.row_buffer = FusedRotaryPositionEncodingContext(self.row_components, max_h)
        self.col_buffer = FusedRotaryPositionEncodingContext(self.col_components, max_w)

    def forward(self, x: torch.Tensor, idx: torch.Tensor) -> torch.Tensor:
        # x: [B, Head, N, C] idx: [N, ]
        B, H, N, C = x.shape
        x0 = x.reshape((-1, N, C))
        return RotaryPE2D.apply(x0, idx, self.row_buffer.cs_components, self.col_buffer.cs_components).reshape(x.shape)
