"""GPU parity of the sliding-window attention on image-layout tensors [B, IH, IW, heads, D]: the
layout the reference's demo converts from and to around the operator (reshape / permute / reshape,
src/tiled_swa.py:753-755).  The token -> pixel map is integer work and must be bit-exact; the
attention results meet the tolerances of the token-layout operator (forward max-abs <= 2e-2,
gradients relative <= 5e-2) and, where the same kernel family runs for both layouts, are bit-equal
to the token-layout result.
"""
import math

import numpy as np
import pytest
import torch

from oracle import attn_oracle as orc

pytestmark = pytest.mark.gpu

FWD_TOL, GRAD_TOL = 2e-2, 5e-2


def _swa():
    from dl_templates_amd import tiled_swa
    return tiled_swa


def _rel(got, want):
    return ((got.float().cpu() - want).abs().max() / want.abs().max().clamp_min(1e-3)).item()


@pytest.mark.parametrize("th,tw,bh,bw,sy,sx", [
    (16, 16, 4, 4, 64 * 8 * 32, 8 * 32), (3, 5, 2, 7, 1000, 3), (7, 1, 1, 1, 9, 9), (1, 9, 5, 1, 11, 13),
    (64, 64, 1, 1, 64 * 64, 64), (5, 3, 8, 8, 1 << 20, 1 << 10), (2, 2, 16, 3, 97, 2), (11, 13, 3, 5, 5 * 13 * 17, 17),
])
def test_token_to_pixel_offsets_are_bit_exact(th, tw, bh, bw, sy, sx):
    got = _swa().swa_image_offsets(th, tw, bh, bw, sy, sx).cpu().numpy()
    assert np.array_equal(got, orc.image_token_offsets(th, tw, bh, bw, sy, sx))


CASES = [
    # B, H, th, tw, bh, bw, WR, WC, dk, dv, dtype, same kernel family for both layouts
    (2, 2, 16, 16, 4, 4, 1, 1, 32, 32, torch.float16, True),     # the reference demo: 4 x 4 pixel tiles, tile mode
    (1, 2, 4, 6, 8, 8, 1, 2, 64, 64, torch.bfloat16, True),      # 64-token tiles, tile mode
    (1, 1, 3, 4, 4, 12, 2, 1, 64, 128, torch.bfloat16, True),    # 48-token tiles, distinct head dims
    (1, 2, 9, 7, 2, 2, 1, 1, 64, 64, torch.bfloat16, False),     # 4-token tiles: generic kernels here, streaming kernels in token layout
    (1, 1, 5, 4, 2, 3, 1, 2, 32, 32, torch.float32, True),       # 6-token tiles, fp32 tensors
    (2, 2, 12, 20, 1, 1, 3, 2, 64, 64, torch.bfloat16, True),    # single-pixel tiles: a plain strided view, token-grid kernels
    (1, 3, 10, 6, 1, 5, 2, 1, 128, 128, torch.bfloat16, False),  # tiles of one pixel row (5 tokens): generic here, streaming in token layout
]


@pytest.mark.parametrize("B,H,th,tw,bh,bw,WR,WC,dk,dv,dtype,same", CASES)
def test_image_layout_forward_backward(B, H, th, tw, bh, bw, WR, WC, dk, dv, dtype, same):
    sw = _swa()
    S, N = bh * bw, th * tw * bh * bw
    q, k, v, do = orc.make_qkv(N + dk + bh, B, H, N, N, dk, dv, dtype)
    scale = 1 / math.sqrt(dk)
    o_w, dq_w, dk_w, dv_w = orc.tiled_swa_grads(q.float(), k.float(), v.float(), do.float(), S, th, tw, WR, WC, scale)
    to_img = lambda t: orc.tokens_to_image(t, th, tw, bh, bw).contiguous()
    qi, ki, vi = (to_img(t).cuda().requires_grad_(True) for t in (q, k, v))
    o = sw.TiledSwaImage.apply(qi, ki, vi, bh, bw, WR, WC, scale)
    o.backward(to_img(do).cuda())
    assert o.shape == (B, th * bh, tw * bw, H, dv) and o.dtype == dtype
    assert (o.float().cpu() - to_img(o_w)).abs().max().item() <= FWD_TOL
    errs = (_rel(qi.grad, to_img(dq_w)), _rel(ki.grad, to_img(dk_w)), _rel(vi.grad, to_img(dv_w)))
    assert max(errs) <= GRAD_TOL, errs
    # the token-layout operator on the permuted copies: the same arithmetic in the same order
    qt, kt, vt = (t.cuda().requires_grad_(True) for t in (q, k, v))
    ot = sw.TiledSwa.apply(qt, kt, vt, S, th, tw, WR, WC, scale)
    ot.backward(do.cuda())
    if same:
        for a, b in ((o, ot), (qi.grad, qt.grad), (ki.grad, kt.grad), (vi.grad, vt.grad)):
            assert torch.equal(a.cpu(), to_img(b.cpu()))


def test_image_views_with_padded_rows_and_packed_heads():
    """q, k, v as slices of one packed projection output [B, IH, IWpad, 3, heads, D] cropped to IW columns:
    pixel rows are not IW pixel columns apart, so even single-pixel tiles need the pixel map."""
    sw = _swa()
    B, H, th, tw, d, pad = 1, 2, 9, 11, 64, 3
    for bh, bw in ((1, 1), (4, 4)):
        S, N = bh * bw, th * tw * bh * bw
        IH, IW = th * bh, tw * bw
        q, k, v, do = orc.make_qkv(7 + bh, B, H, N, N, d, d, torch.bfloat16)
        o_w, dq_w, dk_w, dv_w = orc.tiled_swa_grads(q.float(), k.float(), v.float(), do.float(), S, th, tw, 1, 1, 0.125)
        to_img = lambda t: orc.tokens_to_image(t, th, tw, bh, bw)
        packed = torch.zeros((B, IH, IW + pad, 3, H, d), dtype=torch.bfloat16)
        for j, t in enumerate((q, k, v)):
            packed[:, :, :IW, j] = to_img(t)
        packed = packed.cuda().requires_grad_(True)
        view = packed[:, :, :IW]
        o = sw.TiledSwaImage.apply(view[:, :, :, 0], view[:, :, :, 1], view[:, :, :, 2], bh, bw, 1, 1, 0.125)
        o.backward(to_img(do).cuda())
        assert (o.float().cpu() - to_img(o_w)).abs().max().item() <= FWD_TOL
        g = packed.grad[:, :, :IW]
        errs = (_rel(g[:, :, :, 0], to_img(dq_w)), _rel(g[:, :, :, 1], to_img(dk_w)), _rel(g[:, :, :, 2], to_img(dv_w)))
        assert max(errs) <= GRAD_TOL, errs
        assert packed.grad[:, :, IW:].abs().max().item() == 0.0   # padding columns are never touched


def test_image_entry_rejects_bad_arguments():
    sw = _swa()
    from dl_templates_amd import _lib
    q = torch.zeros((1, 8, 8, 2, 64), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(AssertionError):
        sw.TiledSwaImage.apply(q, q, q, 3, 2, 1, 1, 1.0)            # 8 is not a multiple of 3
    lib = _lib.load()
    shape = _lib.SwaShape(1, 2, 5, 4, 4, 1, 1, 64, 64, 1.0, _lib.dtype_code(q))   # b_size 5 != 2 * 2
    tile = _lib.SwaTile(2, 2)
    lse = torch.zeros((1, 2, 64), dtype=torch.float32, device="cuda")
    rc = lib.dlt_swa_fwd_image(_lib.ptr(q), _lib.strides(q), _lib.ptr(q), _lib.strides(q), _lib.ptr(q), _lib.strides(q),
                               _lib.ptr(q), _lib.strides(q), _lib.ptr(lse), _lib.strides(lse), shape, tile, None,
                               _lib.stream_of(q))
    assert rc == 1 and b"b_size" in lib.dlt_last_error()
    # torch has no negative strides; build them by hand
    import ctypes
    st = (ctypes.c_int64 * 5)(*q.stride())
    st[1] = -st[1]
    shape = _lib.SwaShape(1, 2, 4, 4, 4, 1, 1, 64, 64, 1.0, _lib.dtype_code(q))
    rc = lib.dlt_swa_fwd_image(_lib.ptr(q), st, _lib.ptr(q), _lib.strides(q), _lib.ptr(q), _lib.strides(q),
                               _lib.ptr(q), _lib.strides(q), _lib.ptr(lse), _lib.strides(lse), shape, tile, None,
                               _lib.stream_of(q))
    assert rc == 1 and b"negative stride" in lib.dlt_last_error()


def test_image_layout_with_fused_rotation():
    """The rotary operands stay indexed by the tile-major token number when the tensors are images."""
    from dl_templates_amd import _lib
    sw = _swa()
    B, H, th, tw, bh, bw, d, R = 1, 2, 5, 6, 2, 2, 64, 8
    S, N = bh * bw, th * tw * bh * bw
    q, k, v, do = orc.make_qkv(41, B, H, N, N, d, d, torch.bfloat16)
    idx = torch.cat([orc.make_rope_idx(4, th, tw, 0.1)] * S).reshape(S, -1).t().reshape(-1).contiguous()
    rcs, ccs = orc.rope_tables(R, th), orc.rope_tables(R, tw)
    o_w, dq_w, dk_w, dv_w = orc.rope_swa_grads(q.float(), k.float(), v.float(), do.float(), idx, rcs, ccs, S, th, tw, 1, 1, 0.125)
    to_img = lambda t: orc.tokens_to_image(t, th, tw, bh, bw).contiguous()
    qi, ki, vi, doi = (to_img(t).cuda() for t in (q, k, v, do))
    shape, tile = sw._image_shape(qi, ki, vi, bh, bw, 1, 1, 0.125)
    desc, keep = _lib.rope_desc(idx.cuda(), rcs.cuda(), ccs.cuda())
    o = torch.empty_like(vi)
    lse = torch.empty((B, H, N), dtype=torch.float32, device="cuda")
    lib, P, S_ = _lib.load(), _lib.ptr, _lib.strides
    _lib.check(lib.dlt_swa_fwd_image(P(qi), S_(qi), P(ki), S_(ki), P(vi), S_(vi), P(o), S_(o), P(lse), S_(lse), shape, tile,
                                     desc, _lib.stream_of(qi)))
    assert (o.float().cpu() - to_img(o_w)).abs().max().item() <= FWD_TOL
    dq, dk, dv, delta = torch.empty_like(qi), torch.empty_like(ki), torch.empty_like(vi), torch.empty_like(lse)
    _lib.check(lib.dlt_swa_bwd_image(P(qi), S_(qi), P(ki), S_(ki), P(vi), S_(vi), P(o), S_(o), P(doi), S_(doi),
                                     P(lse), P(delta), S_(lse), P(dq), S_(dq), P(dk), S_(dk), P(dv), S_(dv), shape, tile,
                                     desc, _lib.stream_of(qi)))
    errs = (_rel(dq, to_img(dq_w)), _rel(dk, to_img(dk_w)), _rel(dv, to_img(dv_w)))
    assert max(errs) <= GRAD_TOL, errs
    del keep
