"""GPU parity of the standalone 2D rotary kernel (dlt_rope2d) against the CPU oracle.

Bar: bit-exact for the no-PE mask and for every element the oracle leaves untouched;
rotated elements within 1 bf16 ulp of the fp32-evaluated-then-rounded oracle (in practice
the kernel follows the oracle's evaluation order and the test also reports exact equality).
Shapes follow the reference self-test (src/fused_rope2d.py:230-271: fp32, stride-2 view,
8x8 grid + 16 no-PE tokens) plus mixed no-PE blocks and ragged sizes it never exercises.
"""
import numpy as np
import pytest
import torch

from oracle import attn_oracle as orc

pytestmark = pytest.mark.gpu


def _mods():
    from dl_templates_amd import fused_rope2d
    return fused_rope2d


def _tables(R, h, w, base=10000.0):
    return orc.rope_tables(R, h, base), orc.rope_tables(R, w, base)


def _check(x_cpu, idx, row_cs, col_cs, inverse=False, view=None):
    fr = _mods()
    dev = torch.device("cuda:0")
    xg = x_cpu.to(dev)
    xv = view(xg) if view else xg
    xc = view(x_cpu) if view else x_cpu
    want = orc.rope2d_ref(xc, idx, row_cs, col_cs, inverse=inverse)
    before = xg.clone()
    if inverse:
        fr._launch(xv, idx.to(dev), row_cs.to(dev), col_cs.to(dev), inverse=True)
        got = xv
    else:
        got = fr.RotaryPE2D.apply(xv, idx.to(dev), row_cs.to(dev), col_cs.to(dev))
        assert got.data_ptr() == xv.data_ptr(), "RotaryPE2D must return the same storage"
    got = got.cpu()
    R = row_cs.shape[1]
    # pass-through dims and fully no-PE tokens: bit identical to the input
    bits = orc.pe_mask(idx.numpy())
    untouched = torch.from_numpy(bits == 0)
    assert torch.equal(got[:, untouched], xc[:, untouched])
    assert torch.equal(got[..., 4 * R:], xc[..., 4 * R:])
    if view is not None:
        # elements outside the view must not be written
        full = xg.cpu()
        mask = torch.ones_like(full, dtype=torch.bool)
        view(mask)[...] = False
        assert torch.equal(full[mask], before.cpu()[mask])
    if x_cpu.dtype == torch.float32:
        assert torch.equal(got, want), f"fp32 max diff {(got - want).abs().max()}"
    else:
        ulp = orc.bf16_ulp_diff(got, want) if x_cpu.dtype == torch.bfloat16 else None
        if ulp is not None:
            assert int(ulp.max()) <= 1, f"max bf16 ulp diff {int(ulp.max())}"
        else:
            assert torch.allclose(got.float(), want.float(), atol=2e-3, rtol=2e-3)
    return got, want


def test_pe_mask_bit_exact():
    fr = _mods()
    crafted = np.array([-1, 0, 0xFFFF, 0x7FFF0000 | 5, (3 << 16) | 0xFFFF, (3 << 16) | 0x8000, -65536, -2147483648,
                        0x7FFF7FFF, 1 << 16, (1 << 31) - 1, -65535, 0x00008000], dtype=np.int64).astype(np.int32)
    g = torch.Generator().manual_seed(3)
    rnd = torch.randint(-2**31, 2**31 - 1, (5000,), generator=g, dtype=torch.int64).to(torch.int32).numpy()
    idx = np.concatenate([crafted, rnd])
    got = fr.rope_pe_mask(torch.from_numpy(idx).cuda()).cpu().numpy()
    assert np.array_equal(got, orc.pe_mask(idx))


def test_committed_fixture_bit_equal():
    # tests/golden/rope_16x16.npz (fp32, R = 4, 24 dims of which 16 rotate, row-only / column-only / no-PE tokens):
    # the stored outputs are the bar, the oracle is not called
    import os
    f = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "rope_16x16.npz"))
    fr = _mods()
    idx = torch.from_numpy(f["idx"]).cuda()
    row_cs, col_cs = _tables(4, 16, 16)
    x = torch.from_numpy(f["x"]).cuda()
    y = fr.RotaryPE2D.apply(x, idx, row_cs.cuda(), col_cs.cuda())
    assert y.data_ptr() == x.data_ptr()
    assert np.array_equal(y.cpu().numpy(), f["y"])
    assert np.array_equal(fr.rope_pe_mask(idx).cpu().numpy(), f["pe_bits"])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
def test_c2_shape(dtype):
    # benchmark config 2: B=4, H=8, 64x64 grid, d=64, first 32 dims rotated, 5% no-PE
    torch.manual_seed(0)
    x = torch.randn(32, 4096, 64).to(dtype)
    idx = orc.make_rope_idx(11, 64, 64, 0.05)
    row_cs, col_cs = _tables(8, 64, 64)
    got, want = _check(x, idx, row_cs, col_cs)
    if dtype == torch.bfloat16:
        assert torch.equal(got, want)


def test_inverse_roundtrip_and_inverse_oracle():
    torch.manual_seed(1)
    x = torch.randn(6, 300, 64)
    idx = orc.make_rope_idx(5, 20, 15, 0.1)
    row_cs, col_cs = _tables(8, 20, 15)
    _check(x.clone(), idx, row_cs, col_cs, inverse=True)
    fr = _mods()
    xg = x.cuda()
    y = fr.RotaryPE2D.apply(xg.clone(), idx.cuda(), row_cs.cuda(), col_cs.cuda())
    fr._launch(y, idx.cuda(), row_cs.cuda(), col_cs.cuda(), inverse=True)
    assert torch.allclose(y.cpu(), x, atol=1e-5, rtol=1e-5)


def test_reference_selftest_shape_strided_view_and_autograd():
    # src/fused_rope2d.py:230-271: fp32, q = (x @ W).view(B, N, D, 2)[..., 0] (last stride 2)
    torch.manual_seed(2)
    B, N, D, R, C = 8, 80, 64, 8, 128
    row_b = torch.pow(torch.tensor(1000.0), -2 * (torch.arange(R) / R))
    ang = torch.outer(torch.arange(0, 8).float(), row_b)
    cs = torch.dstack([torch.cos(ang), torch.sin(ang)])
    idx = torch.cat([orc.encode_idx(8, 8), torch.full((16,), -1, dtype=torch.int32)])
    x = torch.randn(B, N, C)
    w = torch.randn(C, D * 2)
    fr = _mods()

    w0 = w.clone().requires_grad_(True)
    q0 = (x @ w0).view(B, N, D, 2)[..., 0]
    o0 = orc.rope2d_ref(q0, idx, cs, cs)
    o0.flatten().sum().backward()

    w1 = w.clone().cuda().requires_grad_(True)
    q1 = (x.cuda() @ w1).view(B, N, D, 2)[..., 0]
    o1 = fr.RotaryPE2D.apply(q1, idx.cuda(), cs.cuda(), cs.cuda())
    o1.flatten().sum().backward()
    assert torch.allclose(o0, o1.cpu(), 1e-2, 1e-2)
    assert torch.allclose(w0.grad, w1.grad.cpu(), 1e-2, 1e-2)
    # tighter than the reference's own tolerance: GEMM on the two devices differs, rotation does not
    assert torch.allclose(o0, o1.cpu(), 1e-4, 1e-4)


@pytest.mark.parametrize("R,C", [(4, 16), (3, 20), (8, 32), (16, 64), (24, 128), (1, 4), (0, 8)])
def test_odd_rdim_and_generic_path(R, C):
    torch.manual_seed(4)
    x = torch.randn(3, 77, C).to(torch.bfloat16)
    idx = orc.make_rope_idx(9, 7, 11, 0.2)
    # axis-only no-PE tokens
    idx[3] = (2 << 16) | 0xFFFF
    idx[4] = (-1 << 16) | 5
    row_cs, col_cs = _tables(R, 7, 11)
    if R == 0:
        row_cs = torch.zeros(7, 0, 2); col_cs = torch.zeros(11, 0, 2)
    _check(x, idx, row_cs, col_cs)


def test_non_contiguous_batch_and_token_strides():
    torch.manual_seed(5)
    base = torch.randn(4, 50, 2, 64).to(torch.bfloat16)
    idx = orc.make_rope_idx(6, 5, 10, 0.1)
    row_cs, col_cs = _tables(8, 5, 10)
    _check(base, idx, row_cs, col_cs, view=lambda t: t[:, :, 1, :])  # token stride 128, vector path
    base2 = torch.randn(50, 4, 65).to(torch.bfloat16)
    _check(base2, idx, row_cs, col_cs, view=lambda t: t.permute(1, 0, 2)[:, :, 1:])  # unaligned -> generic


def test_pair_launch_matches_two_single_launches():
    fr = _mods()
    torch.manual_seed(6)
    q = torch.randn(2, 3, 400, 64).to(torch.bfloat16)
    k = torch.randn(2, 3, 400, 64).to(torch.bfloat16)
    idx = orc.make_rope_idx(7, 20, 20, 0.05)
    row_cs, col_cs = _tables(8, 20, 20)
    wq = orc.rope2d_ref(q.view(-1, 400, 64), idx, row_cs, col_cs).view(q.shape)
    wk = orc.rope2d_ref(k.view(-1, 400, 64), idx, row_cs, col_cs).view(k.shape)
    gq, gk = fr.rope2d_qk_(q.cuda(), k.cuda(), idx.cuda(), row_cs.cuda(), col_cs.cuda())
    assert torch.equal(gq.cpu(), wq) and torch.equal(gk.cpu(), wk)


def test_pair_launch_on_packed_qk_projection():
    """q and k as the two interleaved halves of one fused projection output (the stride-2 views of
    src/fused_rope2d.py:255-259), rotated in ONE launch; the packed tensor is written nowhere else."""
    fr = _mods()
    torch.manual_seed(8)
    B, N, D = 4, 80, 64
    qk = torch.randn(B, N, D, 2).to(torch.bfloat16)
    idx = torch.cat([orc.encode_idx(8, 8), torch.full((16,), -1, dtype=torch.int32)])
    row_cs, col_cs = _tables(8, 8, 8)
    wq = orc.rope2d_ref(qk[..., 0], idx, row_cs, col_cs)
    wk = orc.rope2d_ref(qk[..., 1], idx, row_cs, col_cs)
    g = qk.cuda()
    gq, gk = fr.rope2d_qk_(g[..., 0], g[..., 1], idx.cuda(), row_cs.cuda(), col_cs.cuda())
    assert gq.data_ptr() == g.data_ptr() and gk.data_ptr() == g.data_ptr() + 2
    assert torch.equal(g[..., 0].cpu(), wq) and torch.equal(g[..., 1].cpu(), wk)


def test_module_forward_4d():
    fr = _mods()
    torch.manual_seed(7)
    m = fr.FusedInplaceRotaryPositionEncoding2D(32, 16, 16).cuda()
    x = torch.randn(2, 4, 256, 64).to(torch.bfloat16)
    idx = fr.FusedInplaceRotaryPositionEncoding2D.encode_idx(16, 16)
    assert torch.equal(idx, orc.encode_idx(16, 16))
    want = orc.rope2d_ref(x.view(-1, 256, 64), idx, m.row_buffer.cs_components.cpu(), m.col_buffer.cs_components.cpu())
    got = m(x.cuda(), idx.cuda())
    assert got.shape == x.shape
    assert torch.equal(got.cpu().view(-1, 256, 64), want)
    assert (m.row_buffer.cs_components.cpu() - orc.rope_tables(8, 16)).abs().max().item() <= 1.2e-7


def test_bad_arguments_raise():
    fr = _mods()
    from dl_templates_amd._lib import DltError
    x = torch.randn(2, 10, 16).cuda()
    idx = torch.zeros(10, dtype=torch.int32).cuda()
    cs = orc.rope_tables(8, 4).cuda()  # 4R = 32 > C = 16
    with pytest.raises(DltError):
        fr._launch(x, idx, cs, cs, False)
    with pytest.raises(RuntimeError):
        fr._launch(x.cpu(), idx, cs, cs, False)
