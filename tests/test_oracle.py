"""Pins the CPU oracle (oracle/attn_oracle.py) without a GPU.

The reference holds no golden vectors for this path, so every oracle function is pinned by
what the mathematics fixes: closed-form neighbour counts, brute force on tiny inputs,
reduction to a library routine (dense SDPA) when the window covers the grid, invariants
(row-stochastic P, rotation orthogonality, identity on no-PE tokens) and the committed
fixtures under tests/golden/ (regression anchor for the oracle itself).
"""
import itertools
import math
import os

import numpy as np
import pytest
import torch

from oracle import attn_oracle as orc

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


# ----------------------------------------------------------------------------- a1 neighbour sets
@pytest.mark.parametrize("T,W,count", [(16, 3, 100), (64, 6, 790), (128, 10, 2578), (96, 10, 1906), (160, 10, 3250)])
def test_axis_count_closed_form(T, W, count):
    assert orc.axis_count(T, W) == count
    assert int(orc.neighbor_mask(T, 1, W, 0).sum()) == count


def test_neighbor_mask_bruteforce_all_small_grids():
    for th, tw, wr, wc in itertools.product(range(1, 6), range(1, 6), range(0, 6), range(0, 6)):
        m = orc.neighbor_mask(th, tw, wr, wc)
        want = np.zeros_like(m)
        for r, c, r2, c2 in itertools.product(range(th), range(tw), range(th), range(tw)):
            want[r * tw + c, r2 * tw + c2] = abs(r - r2) <= wr and abs(c - c2) <= wc
        assert np.array_equal(m, want), (th, tw, wr, wc)
        assert np.array_equal(m, m.T)
        assert int(m.sum()) == orc.axis_count(th, wr) * orc.axis_count(tw, wc)
        if wr >= th - 1 and wc >= tw - 1:
            assert m.all()


def test_border_is_truncated_not_shifted():
    m = orc.neighbor_mask(8, 8, 2, 2).reshape(8, 8, 8, 8)
    assert m[0, 0].sum() == 9          # 3x3 corner, a shifted (NATTEN-style) window would give 25
    assert m[4, 4].sum() == 25
    assert m[0, 4].sum() == 15


def test_pairs_match_baseline_table():
    assert orc.swa_pairs(2, 8, 1, 64, 64, 6, 6) == 9_985_600
    assert orc.swa_pairs(1, 16, 1, 128, 128, 10, 10) == 106_337_344
    assert orc.swa_pairs(1, 16, 1, 96, 160, 10, 10) == 99_112_000
    assert orc.swa_pairs(1, 2, 1, 16, 16, 3, 3) == 20_000
    fwd, bwd = orc.attn_flops(9_985_600, 64, 64)
    assert round(fwd / 1e9, 3) == 2.556 and round(bwd / 1e9, 3) == 6.391


# ----------------------------------------------------------------------------- a2 SWA forward
def _qkv(seed, B, H, N, dk, dv):
    return orc.make_qkv(seed, B, H, N, N, dk, dv)


@pytest.mark.parametrize("b_size,th,tw,wr,wc", [(1, 5, 4, 1, 2), (3, 3, 4, 1, 1), (2, 4, 4, 0, 3), (1, 6, 6, 2, 2)])
def test_swa_three_formulations_agree(b_size, th, tw, wr, wc):
    q, k, v, _ = _qkv(1, 1, 2, th * tw * b_size, 8, 5)
    args = (b_size, th, tw, wr, wc, 0.37)
    a = orc.tiled_swa_ref(q, k, v, *args)
    b = orc.tiled_swa_explicit(q, k, v, *args)
    c = orc.tiled_swa_bruteforce(q, k, v, *args).float()
    assert torch.allclose(a, b, atol=2e-6, rtol=1e-5)
    assert torch.allclose(a, c, atol=2e-6, rtol=1e-5)


def test_swa_full_window_equals_dense_sdpa():
    q, k, v, _ = _qkv(2, 2, 2, 36, 16, 8)
    a = orc.tiled_swa_ref(q, k, v, 1, 6, 6, 6, 6, 0.25)
    b = orc.flash_ref(q, k, v, False, 0.25)
    assert torch.allclose(a, b, atol=1e-6, rtol=1e-5)


def test_swa_constant_v_and_row_sums():
    q, k, v, _ = _qkv(3, 1, 1, 64, 8, 4)
    v = torch.ones_like(v) * torch.tensor([1.0, -2.0, 3.0, 0.5])
    o = orc.tiled_swa_ref(q, k, v, 1, 8, 8, 2, 1, 1.0)
    assert torch.allclose(o, v, atol=1e-6)
    _, lse2 = orc.tiled_swa_explicit(q, k, v, 1, 8, 8, 2, 1, 1.0, return_lse2=True)
    s = (q @ k.transpose(-1, -2))
    allowed = torch.from_numpy(orc.token_mask(1, 8, 8, 2, 1))
    p = torch.exp2(s * math.log2(math.e) - lse2[..., None]) * allowed
    assert torch.allclose(p.sum(-1), torch.ones(1, 1, 64), atol=1e-5)


def test_swa_tile_tokens_share_neighbour_set():
    # S > 1 equals S = 1 on the expanded mask (src/tiled_swa.py:713)
    tm = orc.token_mask(3, 2, 3, 1, 1)
    base = orc.neighbor_mask(2, 3, 1, 1)
    assert np.array_equal(tm, np.kron(base, np.ones((3, 3), dtype=bool)))


def test_c1_golden_fixture():
    # benchmark config 1: B=1, H=2, 16x16, d=32, 7x7 window, fp32, scale 1/sqrt(32)
    f = np.load(os.path.join(GOLDEN, "c1_swa_fwd.npz"))
    q, k, v, _ = orc.make_qkv(int(f["seed"]), 1, 2, 256, 256, 32, 32)
    assert np.array_equal(q.numpy(), f["q"]) and np.array_equal(v.numpy(), f["v"])
    o = orc.tiled_swa_ref(q, k, v, 1, 16, 16, 3, 3, 1 / math.sqrt(32))
    assert np.allclose(o.numpy(), f["o"], atol=1e-6, rtol=1e-5)
    # independent route to the same numbers
    o2 = orc.tiled_swa_explicit(q, k, v, 1, 16, 16, 3, 3, 1 / math.sqrt(32))
    assert np.allclose(o2.numpy(), f["o"], atol=2e-6, rtol=1e-5)


# ----------------------------------------------------------------------------- a3/a4 SWA backward
def test_swa_grad_gradcheck_fp64_and_invariants():
    g = torch.Generator().manual_seed(4)
    q, k, v = (torch.randn(1, 1, 12, 4, generator=g, dtype=torch.float64, requires_grad=True) for _ in range(3))
    fn = lambda a, b, c: orc.tiled_swa_explicit(a, b, c, 1, 3, 4, 1, 1, 0.5)
    assert torch.autograd.gradcheck(fn, (q, k, v), eps=1e-6, atol=1e-5)
    q, k, v, do = _qkv(5, 1, 2, 48, 8, 8)
    o, dq, dk, dv = orc.tiled_swa_grads(q, k, v, do, 2, 4, 6, 1, 2, 0.3)
    o2, dq2, dk2, dv2 = orc.tiled_swa_grads(q, k, v, do, 2, 4, 6, 1, 2, 0.3, fn=orc.tiled_swa_explicit)
    for a, b in ((dq, dq2), (dk, dk2), (dv, dv2)):
        assert torch.allclose(a, b, atol=1e-5, rtol=1e-4)
    # softmax logits are invariant to scaling q up and k down: sum(dq*q) == sum(dk*k) per head
    assert torch.allclose((dq * q).sum((-1, -2)), (dk * k).sum((-1, -2)), atol=1e-4, rtol=1e-4)
    # delta closed form: rowsum(P * dP) == rowsum(o * do)
    assert torch.allclose(orc.swa_delta(o, do), (o * do).sum(-1))


# ----------------------------------------------------------------------------- a5 idx decode
def test_idx_decode_crafted_values():
    vals = np.array([-1, 0, 0xFFFF, 0x7FFF0000 | 5, (3 << 16) | 0xFFFF, (3 << 16) | 0x8000, -65536, 1 << 16],
                    dtype=np.int64).astype(np.int32)
    row, col = orc.decode_idx(vals)
    assert row.tolist() == [-1, 0, 0, 0x7FFF, 3, 3, -1, 1]
    assert col.tolist() == [-1, 0, -1, 5, -1, -32768, 0, 0]
    assert orc.pe_mask(vals).tolist() == [0, 3, 1, 3, 1, 1, 2, 3]
    e = orc.encode_idx(3, 5)
    r, c = orc.decode_idx(e.numpy())
    assert r.reshape(3, 5)[2, 4] == 2 and c.reshape(3, 5)[2, 4] == 4 and e.dtype == torch.int32
    # the eager reference decodes with ((idx >> 16) & 0xFFFF).to(int16): same 16-bit values
    t = torch.from_numpy(vals)
    assert np.array_equal(((t >> 16) & 0xFFFF).to(torch.int16).numpy(), row)
    assert np.array_equal((t & 0xFFFF).to(torch.int16).numpy(), col)


# ----------------------------------------------------------------------------- a6 rotation
def test_rope_is_a_rotation_and_identity_on_nope():
    g = torch.Generator().manual_seed(6)
    x = torch.randn(3, 40, 24, generator=g)
    idx = orc.make_rope_idx(7, 5, 8, 0.2)
    idx[0] = (1 << 16) | 0xFFFF   # row only
    idx[1] = (-1 << 16) | 3       # col only
    idx[2] = -1
    R = 4
    rcs, ccs = orc.rope_tables(R, 5), orc.rope_tables(R, 8)
    y = orc.rope2d_ref(x, idx, rcs, ccs)
    assert torch.equal(y[..., 4 * R:], x[..., 4 * R:])
    assert torch.equal(y[:, 2], x[:, 2])
    assert torch.equal(y[:, 0, 2 * R:], x[:, 0, 2 * R:]) and not torch.equal(y[:, 0, :2 * R], x[:, 0, :2 * R])
    assert torch.equal(y[:, 1, :2 * R], x[:, 1, :2 * R])
    # norm of every rotated pair is preserved; inverse undoes forward
    n0 = x[..., :R] ** 2 + x[..., R:2 * R] ** 2
    n1 = y[..., :R] ** 2 + y[..., R:2 * R] ** 2
    assert torch.allclose(n0, n1, atol=1e-5)
    assert torch.allclose(orc.rope2d_bwd_ref(y, idx, rcs, ccs), x, atol=1e-6)
    # token (r, c): the pair (i, i+R) turns by r * theta_i: check one by hand with complex numbers
    r, c = 3, 6
    n = r * 8 + c
    if idx[n] >= 0:
        th = 10000.0 ** (-2 * np.arange(R) / R)
        z = (x[0, n, :R].double().numpy() + 1j * x[0, n, R:2 * R].double().numpy()) * np.exp(1j * r * th)
        assert np.allclose(z.real, y[0, n, :R].numpy(), atol=1e-5) and np.allclose(z.imag, y[0, n, R:2 * R].numpy(), atol=1e-5)
        z = (x[0, n, 2 * R:3 * R].double().numpy() + 1j * x[0, n, 3 * R:4 * R].double().numpy()) * np.exp(1j * c * th)
        assert np.allclose(z.real, y[0, n, 2 * R:3 * R].numpy(), atol=1e-5)


def test_rope_backward_is_autograd_of_forward():
    g = torch.Generator().manual_seed(8)
    x = torch.randn(2, 12, 16, generator=g, requires_grad=True)
    idx = orc.make_rope_idx(9, 3, 4, 0.3)
    rcs, ccs = orc.rope_tables(4, 3), orc.rope_tables(4, 4)
    do = torch.randn(2, 12, 16, generator=g)
    orc.rope2d_ref(x, idx, rcs, ccs).backward(do)
    assert torch.allclose(x.grad, orc.rope2d_bwd_ref(do, idx, rcs, ccs), atol=1e-6)


def test_rope_tables_match_the_reference_self_test_construction():
    """The only table construction in the reference is its self-test, src/fused_rope2d.py:236-246; it is typed
    here as those lines have it (fp32 torch ops, base 1000, R = 8, 8 positions) and compared with the oracle's
    generator and with the product's table holder.  A schedule of another form (exponent -i/R, another base, sin
    and cos swapped, [R, len] instead of [len, R]) fails."""
    from dl_templates_amd.rope2d import FusedRotaryPositionEncodingContext as Ctx
    for n_rdim, n_max in ((8, 8), (4, 33), (16, 64)):
        bases = torch.pow(1000, -2 * (torch.arange(n_rdim) / n_rdim))
        indices = torch.arange(0, n_max)
        cos_c = torch.cos(torch.outer(indices, bases))
        sin_c = torch.sin(torch.outer(indices, bases))
        literal = torch.dstack([cos_c, sin_c])
        assert literal.shape == (n_max, n_rdim, 2)
        mine = orc.rope_tables(n_rdim, n_max, base=1000.0)
        prod = Ctx(2 * n_rdim, n_max, base=1000.0).cs_components
        assert mine.shape == literal.shape and prod.shape == literal.shape and prod.dtype == torch.float32
        # the literal expression forms its angles in fp32: half an ulp of the largest angle (< 64) is 4e-6
        assert (mine - literal).abs().max().item() <= 8e-6
        assert (prod - literal).abs().max().item() <= 8e-6
        # oracle (complex exponential) and product (cos / sin), both from float64 angles, agree to an fp32 ulp
        assert (mine - prod).abs().max().item() <= 1.2e-7
        other_form = torch.cos(torch.outer(indices.double(), torch.pow(torch.tensor(1000.0, dtype=torch.float64), -(torch.arange(n_rdim) / n_rdim))))
        assert (mine[..., 0].double() - other_form).abs().max().item() > 1e-2


def test_rope_tables_identities():
    # unit circle; position p is p steps of position 1 (angle addition); position 0 is the identity
    t = orc.rope_tables(8, 40).double()
    assert torch.allclose(t[..., 0] ** 2 + t[..., 1] ** 2, torch.ones(40, 8, dtype=torch.float64), atol=1e-6)
    z = torch.complex(t[..., 0], t[..., 1])
    assert torch.allclose(z[17] * z[5], z[22], atol=1e-6) and torch.allclose(z[1] ** 3, z[3], atol=1e-6)
    # successive pairs slow down by the constant factor base ** (-2 / R)
    ang = torch.atan2(t[1, :, 1], t[1, :, 0])
    assert torch.allclose(ang[1:] / ang[:-1], torch.full((7,), 10000.0 ** (-2 / 8), dtype=torch.float64), rtol=1e-5)


def test_rope_table_packing_and_golden():
    t = orc.rope_tables(8, 64)
    assert t.shape == (64, 8, 2) and t.dtype == torch.float32
    assert torch.equal(t[0, :, 0], torch.ones(8)) and torch.equal(t[0, :, 1], torch.zeros(8))
    assert abs(float(t[1, 0, 0]) - math.cos(1.0)) < 1e-7 and abs(float(t[1, 0, 1]) - math.sin(1.0)) < 1e-7
    f = np.load(os.path.join(GOLDEN, "rope_16x16.npz"))
    idx = torch.from_numpy(f["idx"])
    x = torch.from_numpy(f["x"])
    y = orc.rope2d_ref(x, idx, orc.rope_tables(4, 16), orc.rope_tables(4, 16))
    assert np.array_equal(y.numpy(), f["y"])
    assert np.array_equal(orc.pe_mask(f["idx"]), f["pe_bits"])


# ----------------------------------------------------------------------------- a9/a10 flash
def test_flash_ref_matches_explicit_softmax_lq_ne_lk():
    q, k, v, do = orc.make_qkv(10, 1, 2, 20, 33, 8, 12)
    o = orc.flash_ref(q, k, v, False, 0.4)
    p = torch.softmax(q @ k.transpose(-1, -2) * 0.4, -1)
    assert torch.allclose(o, p @ v, atol=1e-6)
    lse2 = orc.flash_lse2(q, k, 0.4)
    assert torch.allclose(torch.exp2(q @ k.transpose(-1, -2) * 0.4 * math.log2(math.e) - lse2[..., None]), p, atol=1e-6)
    o2, dq, dk, dv = orc.flash_grads(q, k, v, do, False, 0.4)
    assert torch.allclose(dv, p.transpose(-1, -2) @ do, atol=1e-5)


def test_flash_lse2_causal_is_the_log_sum_over_keys_up_to_the_query():
    # per-row evaluation with explicit key lists: a flipped or shifted mask changes the first rows
    q, k, v, do = orc.make_qkv(14, 1, 2, 17, 17, 8, 8)
    scale = 0.7
    got = orc.flash_lse2(q, k, scale, causal=True)
    s = (q @ k.transpose(-1, -2)) * scale
    for i in range(17):
        want = torch.logsumexp(s[..., i, : i + 1], dim=-1) / math.log(2.0)
        assert torch.allclose(got[..., i], want, atol=1e-5), i
        if 0 < i < 16:
            # the transposed mask (keys from the query on) and the strict one (keys before the query) give other values
            for wrong in (s[..., i, i:], s[..., i, :i]):
                assert not torch.allclose(got[..., i], torch.logsumexp(wrong, dim=-1) / math.log(2.0), atol=1e-3)
    # row 0 sees one key: lse2 is that score in the log2 domain
    assert torch.allclose(got[..., 0], s[..., 0, 0] * math.log2(math.e), atol=1e-5)
    # exp2(s2 - lse2) over the visible keys are the softmax rows SDPA's causal mode uses
    p = torch.exp2(s * math.log2(math.e) - got[..., None]).tril()
    assert torch.allclose(p.sum(-1), torch.ones(1, 2, 17), atol=1e-5)
    o = orc.flash_ref(q, k, v, True, scale)
    assert torch.allclose(p @ v, o, atol=1e-5)
    # and it differs from the dense one everywhere but in the last row
    dense = orc.flash_lse2(q, k, scale, causal=False)
    assert torch.allclose(got[..., -1], dense[..., -1], atol=1e-5)
    assert (got[..., :-1] < dense[..., :-1] - 1e-4).all()


def test_composed_rope_swa_grads_are_autograd_of_composition():
    q, k, v, do = orc.make_qkv(12, 1, 1, 16, 16, 16, 8)
    idx = orc.make_rope_idx(13, 4, 4, 0.2)
    rcs, ccs = orc.rope_tables(4, 4), orc.rope_tables(4, 4)
    args = (idx, rcs, ccs, 1, 4, 4, 1, 1, 0.25)
    o, dq, dk, dv = orc.rope_swa_grads(q, k, v, do, *args)
    qa, ka, va = (t.clone().requires_grad_(True) for t in (q, k, v))
    oa = orc.rope_swa_ref(qa, ka, va, *args)
    oa.backward(do)
    assert torch.allclose(o, oa.detach(), atol=1e-6)
    assert torch.allclose(dq, qa.grad, atol=1e-5) and torch.allclose(dk, ka.grad, atol=1e-5)
    assert torch.allclose(dv, va.grad, atol=1e-5)


# ---- layout adapters (src/tiled_swa.py:753-755) -------------------------------------------------
@pytest.mark.parametrize("th,tw,bh,bw", [(2, 3, 4, 4), (3, 2, 2, 5), (4, 5, 1, 1), (1, 4, 3, 1), (5, 1, 1, 7)])
def test_image_layout_three_formulations_agree(th, tw, bh, bw):
    """reshape/permute (the reference's text), the closed-form index and plain loops give one map."""
    B, H, D = 2, 3, 4
    N = th * tw * bh * bw
    x = torch.arange(B * H * N * D, dtype=torch.float32).reshape(B, H, N, D)
    img = orc.tokens_to_image(x, th, tw, bh, bw)
    assert img.shape == (B, th * bh, tw * bw, H, D)
    assert torch.equal(orc.image_to_tokens(img, th, tw, bh, bw), x)          # inverse
    index = orc.image_token_index(th, tw, bh, bw)
    assert sorted(index.reshape(-1).tolist()) == list(range(N))               # a permutation
    for y in range(th * bh):                                                  # loops: tile, then pixel inside the tile
        for xx in range(tw * bw):
            tile = (y // bh) * tw + xx // bw
            n = tile * bh * bw + (y % bh) * bw + xx % bw
            assert index[y, xx] == n
            assert torch.equal(img[:, y, xx], x[:, :, n])
    sy, sx = 1000, 7
    off = orc.image_token_offsets(th, tw, bh, bw, sy, sx)
    for n in (0, N // 2, N - 1):
        y, xx = np.argwhere(index == n)[0]
        assert off[n] == y * sy + xx * sx


def test_image_layout_attention_commutes_with_the_adapter():
    """Attention on tokens and on the image are the same numbers in two layouts; the tiles of the image
    are bh x bw pixel blocks whose neighbour sets are those of the tile grid."""
    th, tw, bh, bw, H, d = 3, 4, 2, 2, 2, 8
    q, k, v, _ = orc.make_qkv(5, 1, H, th * tw * bh * bw, th * tw * bh * bw, d, d)
    o = orc.tiled_swa_ref(q, k, v, bh * bw, th, tw, 1, 1, 0.3)
    o_img = orc.tokens_to_image(o, th, tw, bh, bw)
    # pixel (y, x) attends pixel (y', x') iff their tiles are neighbours: brute force on the image
    qi, ki, vi = (orc.tokens_to_image(t, th, tw, bh, bw) for t in (q, k, v))
    for (y, x) in [(0, 0), (3, 5), (5, 7), (2, 2)]:
        ys = [yy for yy in range(th * bh) if abs(yy // bh - y // bh) <= 1]
        xs = [xx for xx in range(tw * bw) if abs(xx // bw - x // bw) <= 1]
        for h in range(H):
            keys = torch.stack([ki[0, yy, xx, h] for yy in ys for xx in xs])
            vals = torch.stack([vi[0, yy, xx, h] for yy in ys for xx in xs])
            p = torch.softmax(keys @ qi[0, y, x, h] * 0.3, dim=0)
            assert torch.allclose(p @ vals, o_img[0, y, x, h], atol=1e-5)
