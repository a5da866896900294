"""GPU parity of flash attention (dlt_flash_fwd / dlt_flash_bwd) against SDPA on the CPU.

Follows the reference's own check (src/flash_attn.py:616-659: q, k L2-normalised, loss =
o.sum(), allclose(1e-2, 1e-2) on o, dq, dk, dv, Z=4, H in {4,8}, N in {512,2048},
dv in {16,32}, dk in {16,64}) with seeded inputs, plus Lq != Lk, odd lengths, bf16 and the
stated tolerances (forward max-abs <= 2e-2, gradients relative <= 5e-2).
"""
import itertools
import math

import pytest
import torch

from oracle import attn_oracle as orc

pytestmark = pytest.mark.gpu


def _fa():
    from dl_templates_amd import flash_attn
    return flash_attn


def _l2(x):
    return x / torch.linalg.norm(x, dim=-1, keepdims=True)


def _rel(got, want):
    return ((got.float().cpu() - want).abs().max() / want.abs().max().clamp_min(1e-3)).item()


SWEEP = list(itertools.product([False, True], [4, 8], [512, 2048], [16, 32], [16, 64]))


@pytest.mark.parametrize("causal,head,n_ctx,h_dim,k_dim", SWEEP[::3] + [SWEEP[-1]])
def test_reference_correctness_sweep(causal, head, n_ctx, h_dim, k_dim):
    Z = 2 if n_ctx == 2048 else 4
    g = torch.Generator().manual_seed(n_ctx + head + h_dim + k_dim)
    q = _l2(torch.randn((Z, head, n_ctx, k_dim), generator=g)).half()
    k = _l2(torch.randn((Z, head, n_ctx, k_dim), generator=g)).half()
    v = torch.randn((Z, head, n_ctx, h_dim), generator=g).half()
    do = torch.ones((Z, head, n_ctx, h_dim))
    o_std, dq, dk, dv = orc.flash_grads(q.float(), k.float(), v.float(), do, causal, 1.0)
    q2, k2, v2 = (t.cuda().requires_grad_(True) for t in (q, k, v))
    o = _fa().attention(q2, k2, v2, causal, 1.0)
    o.flatten().sum().backward()
    assert torch.allclose(o.float().cpu(), o_std, atol=1e-2, rtol=1e-2)
    assert torch.allclose(q2.grad.float().cpu(), dq, atol=1e-2, rtol=1e-2)
    assert torch.allclose(k2.grad.float().cpu(), dk, atol=1e-2, rtol=1e-2)
    assert torch.allclose(v2.grad.float().cpu(), dv, atol=1e-2, rtol=1e-2)


@pytest.mark.parametrize("Lq,Lk,dk,dv,dtype", [
    (256, 512, 64, 128, torch.bfloat16), (100, 333, 64, 128, torch.bfloat16), (1, 1, 16, 16, torch.bfloat16),
    (129, 31, 32, 64, torch.float16), (64, 1000, 128, 128, torch.bfloat16), (300, 300, 64, 64, torch.float32),
    (17, 257, 48, 80, torch.bfloat16)])
def test_cross_attention_distinct_dims_and_lengths(Lq, Lk, dk, dv, dtype):
    q, k, v, do = orc.make_qkv(Lq * 7 + Lk, 2, 3, Lq, Lk, dk, dv, dtype)
    scale = 1 / math.sqrt(dk)
    o_w, dq_w, dk_w, dv_w = orc.flash_grads(q.float(), k.float(), v.float(), do.float(), False, scale)
    qg, kg, vg = (t.cuda().requires_grad_(True) for t in (q, k, v))
    o = _fa().attention(qg, kg, vg, False, scale)
    o.backward(do.cuda())
    assert o.shape == (2, 3, Lq, dv) and o.dtype == dtype
    assert (o.float().cpu() - o_w).abs().max().item() <= 2e-2
    errs = (_rel(qg.grad, dq_w), _rel(kg.grad, dk_w), _rel(vg.grad, dv_w))
    assert max(errs) <= 5e-2, errs


@pytest.mark.parametrize("causal,Lq,Lk,dk,dv,dtype", [
    (False, 256, 512, 64, 128, torch.bfloat16), (False, 100, 333, 64, 64, torch.float16), (True, 300, 300, 128, 128, torch.bfloat16),
    (True, 129, 129, 32, 32, torch.float16), (False, 77, 190, 48, 80, torch.float32), (False, 1, 1, 16, 16, torch.bfloat16)])
def test_saved_log_sum_exp(causal, Lq, Lk, dk, dv, dtype):
    """M = m + log2(l), the vector the forward pass saves for the backward pass (src/flash_attn.py:168-171),
    directly against the oracle; 2e-2 in log2 units."""
    q, k, v, _ = orc.make_qkv(Lq + 3 * Lk, 2, 2, Lq, Lk, dk, dv, dtype)
    scale = 1 / math.sqrt(dk)
    o, M = _fa()._forward(q.cuda(), k.cuda(), v.cuda(), causal, scale)
    assert M.dtype == torch.float32 and M.shape == (2, 2, Lq)
    want = orc.flash_lse2(q, k, scale, causal)
    assert (M.cpu() - want).abs().max().item() <= 2e-2
    assert (o.float().cpu() - orc.flash_ref(q.float(), k.float(), v.float(), causal, scale)).abs().max().item() <= 2e-2


def test_negative_scale_matches_sdpa():
    q, k, v, do = orc.make_qkv(91, 1, 2, 200, 320, 64, 64, torch.bfloat16)
    o_w, dq_w, dk_w, dv_w = orc.flash_grads(q.float(), k.float(), v.float(), do.float(), False, -0.125)
    qg, kg, vg = (t.cuda().requires_grad_(True) for t in (q, k, v))
    o = _fa().attention(qg, kg, vg, False, -0.125)
    o.backward(do.cuda())
    assert (o.float().cpu() - o_w).abs().max().item() <= 2e-2
    assert max(_rel(qg.grad, dq_w), _rel(kg.grad, dk_w), _rel(vg.grad, dv_w)) <= 5e-2


@pytest.mark.parametrize("causal,Lq,Lk,dk,dv,dtype", [
    (False, 256, 384, 256, 256, torch.bfloat16), (True, 200, 200, 256, 256, torch.float16), (False, 65, 130, 256, 64, torch.bfloat16),
    (False, 100, 100, 64, 256, torch.float16), (True, 129, 129, 192, 160, torch.bfloat16), (False, 40, 70, 256, 256, torch.float32)])
def test_head_dim_256(causal, Lq, Lk, dk, dv, dtype):
    """The reference admits head dims up to 256 (src/flash_attn.py:460-462); forward, saved log-sum-exp and
    gradients against SDPA."""
    q, k, v, do = orc.make_qkv(Lq + dk, 1, 2, Lq, Lk, dk, dv, dtype)
    scale = 1 / math.sqrt(dk)
    o_w, dq_w, dk_w, dv_w = orc.flash_grads(q.float(), k.float(), v.float(), do.float(), causal, scale)
    qg, kg, vg = (t.cuda().requires_grad_(True) for t in (q, k, v))
    o = _fa().attention(qg, kg, vg, causal, scale)
    o.backward(do.cuda())
    assert o.shape == (1, 2, Lq, dv) and o.dtype == dtype
    assert (o.float().cpu() - o_w).abs().max().item() <= 2e-2
    errs = (_rel(qg.grad, dq_w), _rel(kg.grad, dk_w), _rel(vg.grad, dv_w))
    assert max(errs) <= 5e-2, errs
    _, M = _fa()._forward(q.cuda(), k.cuda(), v.cuda(), causal, scale)
    assert (M.cpu() - orc.flash_lse2(q, k, scale, causal)).abs().max().item() <= 2e-2


def test_c5_shape_reduced_batch():
    # benchmark config 5 shape with B=1, H=2 (CPU oracle time): Lq=4096, Lk=8192, 64/128
    q, k, v, do = orc.make_qkv(55, 1, 2, 4096, 8192, 64, 128, torch.bfloat16)
    o_w, dq_w, dk_w, dv_w = orc.flash_grads(q.float(), k.float(), v.float(), do.float(), False, 0.125)
    qg, kg, vg = (t.cuda().requires_grad_(True) for t in (q, k, v))
    o = _fa().attention(qg, kg, vg, False, 0.125)
    o.backward(do.cuda())
    assert (o.float().cpu() - o_w).abs().max().item() <= 2e-2
    errs = (_rel(qg.grad, dq_w), _rel(kg.grad, dk_w), _rel(vg.grad, dv_w))
    print("c5 rel errs", errs)
    assert max(errs) <= 5e-2, errs


def test_causal_matches_sdpa_bf16():
    q, k, v, do = orc.make_qkv(56, 1, 2, 777, 777, 64, 64, torch.bfloat16)
    o_w, dq_w, dk_w, dv_w = orc.flash_grads(q.float(), k.float(), v.float(), do.float(), True, 0.125)
    qg, kg, vg = (t.cuda().requires_grad_(True) for t in (q, k, v))
    o = _fa().attention(qg, kg, vg, True, 0.125)
    o.backward(do.cuda())
    assert (o.float().cpu() - o_w).abs().max().item() <= 2e-2
    assert max(_rel(qg.grad, dq_w), _rel(kg.grad, dk_w), _rel(vg.grad, dv_w)) <= 5e-2


@pytest.mark.parametrize("N,dk,dv,dtype", [
    (1, 64, 64, torch.bfloat16), (63, 64, 128, torch.bfloat16), (64, 128, 128, torch.bfloat16),
    (65, 64, 64, torch.float16), (129, 64, 128, torch.bfloat16), (1000, 128, 128, torch.bfloat16),
    (384, 32, 32, torch.float16)])
def test_causal_lengths_and_dims(N, dk, dv, dtype):
    """Causal fast path: lengths around the 64-key chunk and the 128-query block, all head-dim classes."""
    q, k, v, do = orc.make_qkv(N + dk, 2, 2, N, N, dk, dv, dtype)
    scale = 1 / math.sqrt(dk)
    o_w, dq_w, dk_w, dv_w = orc.flash_grads(q.float(), k.float(), v.float(), do.float(), True, scale)
    qg, kg, vg = (t.cuda().requires_grad_(True) for t in (q, k, v))
    o = _fa().attention(qg, kg, vg, True, scale)
    o.backward(do.cuda())
    assert (o.float().cpu() - o_w).abs().max().item() <= 2e-2
    errs = (_rel(qg.grad, dq_w), _rel(kg.grad, dk_w), _rel(vg.grad, dv_w))
    assert max(errs) <= 5e-2, errs


@pytest.mark.parametrize("B,H,N,dk,dv", [(1, 7, 4096, 128, 128), (3, 3, 2048, 64, 64), (1, 5, 1536, 64, 128)])
def test_causal_block_order_over_heads(B, H, N, dk, dv):
    """Under a causal mask the workgroups of several (batch, head) slabs are interleaved, heaviest blocks first, in groups
    sized by their K / V footprint (groups of 2, 8 and 7 heads here, the last one partial).  The order must not change any
    result: every slab run on its own (one head per call) gives the same bits, and slab 0 matches the oracle."""
    q, k, v, do = orc.make_qkv(N + H, B, H, N, N, dk, dv, torch.bfloat16)
    scale = 1 / math.sqrt(dk)
    qg, kg, vg = (t.cuda().requires_grad_(True) for t in (q, k, v))
    o = _fa().attention(qg, kg, vg, True, scale)
    o.backward(do.cuda())
    for b in range(B):
        for h in range(H):
            q1, k1, v1 = (t[b:b + 1, h:h + 1].contiguous().cuda().requires_grad_(True) for t in (q, k, v))
            o1 = _fa().attention(q1, k1, v1, True, scale)
            o1.backward(do[b:b + 1, h:h + 1].contiguous().cuda())
            assert torch.equal(o1[0, 0], o[b, h]), (b, h)
            assert torch.equal(q1.grad[0, 0], qg.grad[b, h]) and torch.equal(k1.grad[0, 0], kg.grad[b, h]) \
                and torch.equal(v1.grad[0, 0], vg.grad[b, h]), (b, h)
    sl = (slice(0, 1), slice(0, 1))
    o_w, dq_w, dk_w, dv_w = orc.flash_grads(q[sl].float(), k[sl].float(), v[sl].float(), do[sl].float(), True, scale)
    assert (o[sl].float().cpu() - o_w).abs().max().item() <= 2e-2
    assert max(_rel(qg.grad[sl], dq_w), _rel(kg.grad[sl], dk_w), _rel(vg.grad[sl], dv_w)) <= 5e-2


@pytest.mark.parametrize("causal,dk,dv,dtype", [
    (False, 64, 128, torch.bfloat16), (False, 64, 64, torch.float16), (False, 128, 128, torch.bfloat16),
    (True, 64, 128, torch.float16), (True, 128, 128, torch.bfloat16), (True, 64, 64, torch.bfloat16)])
def test_chunk_boundaries_of_the_async_staged_kernels(causal, dk, dv, dtype):
    """Head dims of exactly 64 / 128 run on the kernels that copy chunks HBM -> LDS asynchronously into two or three
    buffers: lengths of one, two, three and four chunks (64 keys in the backward kernels, 128 in the forward kernel),
    one token more and one less, and query counts around the 128- and 256-query workgroups."""
    pairs = [(1, 1), (63, 64), (200, 65), (128, 127), (129, 128), (256, 129), (257, 191), (130, 192), (70, 193), (255, 256),
             (33, 257), (300, 320)]
    scale = 1 / math.sqrt(dk)
    for Lq, Lk in pairs:
        if causal:
            Lq = Lk
        q, k, v, do = orc.make_qkv(Lq * 5 + Lk + dk, 1, 2, Lq, Lk, dk, dv, dtype)
        o_w, dq_w, dk_w, dv_w = orc.flash_grads(q.float(), k.float(), v.float(), do.float(), causal, scale)
        qg, kg, vg = (t.cuda().requires_grad_(True) for t in (q, k, v))
        o = _fa().attention(qg, kg, vg, causal, scale)
        o.backward(do.cuda())
        assert (o.float().cpu() - o_w).abs().max().item() <= 2e-2, (Lq, Lk)
        errs = (_rel(qg.grad, dq_w), _rel(kg.grad, dk_w), _rel(vg.grad, dv_w))
        assert max(errs) <= 5e-2, (Lq, Lk, errs)


@pytest.mark.parametrize("causal,dk,dv,dtype", [
    (False, 40, 40, torch.bfloat16), (True, 48, 80, torch.float16), (False, 80, 80, torch.bfloat16), (True, 96, 96, torch.bfloat16),
    (False, 72, 120, torch.float16), (False, 56, 128, torch.bfloat16), (True, 128, 104, torch.bfloat16), (False, 64, 8, torch.float16)])
def test_async_staged_kernels_with_head_dims_below_the_padded_class(causal, dk, dv, dtype):
    """Head dims that are multiples of 8 below their class (64 or 128) also run on the asynchronously staged kernels: the
    lanes of the missing 16-byte pieces copy nothing and their LDS slots are zeroed once.  Lengths of one to several
    chunks, one token more and less."""
    scale = 1 / math.sqrt(dk)
    for Lq, Lk in [(1, 1), (65, 64), (130, 191), (257, 320), (300, 129), (512, 513)]:
        if causal:
            Lq = Lk
        q, k, v, do = orc.make_qkv(Lq + 3 * Lk + dk + dv, 2, 2, Lq, Lk, dk, dv, dtype)
        o_w, dq_w, dk_w, dv_w = orc.flash_grads(q.float(), k.float(), v.float(), do.float(), causal, scale)
        qg, kg, vg = (t.cuda().requires_grad_(True) for t in (q, k, v))
        o = _fa().attention(qg, kg, vg, causal, scale)
        o.backward(do.cuda())
        assert (o.float().cpu() - o_w).abs().max().item() <= 2e-2, (Lq, Lk)
        errs = (_rel(qg.grad, dq_w), _rel(kg.grad, dk_w), _rel(vg.grad, dv_w))
        assert max(errs) <= 5e-2, (Lq, Lk, errs)


@pytest.mark.parametrize("causal,dk,dv,dtype", [(False, 100, 100, torch.bfloat16), (True, 50, 36, torch.float16), (False, 20, 127, torch.bfloat16),
                                                 (True, 1, 3, torch.float16), (False, 65, 9, torch.bfloat16)])
def test_head_dims_that_are_not_multiples_of_eight(causal, dk, dv, dtype):
    """The public entry pads such head dims with zero columns to the next multiple of 8 (the kernels read 16-byte row
    pieces) and slices the results: shapes, contiguity and values against the oracle."""
    scale = 1 / math.sqrt(dk)
    for Lq, Lk in [(1, 1), (130, 191), (300, 129)]:
        if causal:
            Lq = Lk
        q, k, v, do = orc.make_qkv(Lq + Lk + dk + dv, 1, 3, Lq, Lk, dk, dv, dtype)
        o_w, dq_w, dk_w, dv_w = orc.flash_grads(q.float(), k.float(), v.float(), do.float(), causal, scale)
        qg, kg, vg = (t.cuda().requires_grad_(True) for t in (q, k, v))
        o = _fa().attention(qg, kg, vg, causal, scale)
        o.backward(do.cuda())
        assert o.shape == o_w.shape and o.is_contiguous()
        assert qg.grad.shape == q.shape and kg.grad.shape == k.shape and vg.grad.shape == v.shape
        assert (o.float().cpu() - o_w).abs().max().item() <= 2e-2, (Lq, Lk)
        errs = (_rel(qg.grad, dq_w), _rel(kg.grad, dk_w), _rel(vg.grad, dv_w))
        assert max(errs) <= 5e-2, (Lq, Lk, errs)


@pytest.mark.parametrize("causal,dk,dv", [(False, 64, 128), (False, 128, 128), (True, 128, 128), (True, 64, 64)])
def test_async_staged_kernels_repeat_bit_for_bit(causal, dk, dv):
    """The kernels are deterministic, so a chunk read before its asynchronous copy has landed (or overwritten while it is
    still being read) shows as a difference between repeats: 25 forward + backward passes over many chunks (two chunk
    buffers at 64/128 forward and at 128/128, three elsewhere) must all equal the first, bit for bit."""
    B, H, L = 2, 8, 4096
    q, k, v, do = (t.cuda() for t in orc.make_qkv(77, B, H, L, L, dk, dv, torch.bfloat16))
    scale = 1 / math.sqrt(dk)
    first = None
    for _ in range(25):
        qg, kg, vg = (t.detach().requires_grad_(True) for t in (q, k, v))
        o, M = _fa()._forward(qg.detach(), kg.detach(), vg.detach(), causal, scale)
        o2 = _fa().attention(qg, kg, vg, causal, scale)
        o2.backward(do)
        got = (o, M, o2.detach(), qg.grad, kg.grad, vg.grad)
        if first is None:
            first = got
        else:
            for a, b in zip(first, got):
                assert torch.equal(a, b)


@pytest.mark.parametrize("causal", [False, True])
def test_views_of_a_packed_projection(causal):
    """q, k, v as strided views of one packed [B, L, H, dk + dk + dv] projection output (token stride H (2 dk + dv), head
    stride 2 dk + dv) and a transposed upstream gradient: the asynchronously staged kernels address tokens by stride."""
    B, H, L, dk, dv = 2, 3, 200, 64, 128
    g = torch.Generator().manual_seed(11)
    packed = torch.randn(B, L, H, 2 * dk + dv, generator=g).to(torch.bfloat16)
    do = torch.randn(B, L, H, dv, generator=g).to(torch.bfloat16)
    scale = 1 / math.sqrt(dk)
    views = lambda t: (t[..., :dk].permute(0, 2, 1, 3), t[..., dk:2 * dk].permute(0, 2, 1, 3), t[..., 2 * dk:].permute(0, 2, 1, 3))
    q, k, v = views(packed)
    o_w, dq_w, dk_w, dv_w = orc.flash_grads(q.float().contiguous(), k.float().contiguous(), v.float().contiguous(),
                                            do.permute(0, 2, 1, 3).float().contiguous(), causal, scale)
    pg = packed.cuda().requires_grad_(True)
    qg, kg, vg = views(pg)
    assert not qg.is_contiguous()
    o = _fa().attention(qg, kg, vg, causal, scale)
    o.backward(do.cuda().permute(0, 2, 1, 3))
    assert (o.float().cpu() - o_w).abs().max().item() <= 2e-2
    got = views(pg.grad)
    errs = (_rel(got[0], dq_w), _rel(got[1], dk_w), _rel(got[2], dv_w))
    assert max(errs) <= 5e-2, errs


def test_bad_arguments_raise():
    from dl_templates_amd._lib import DltError
    q = torch.randn(1, 1, 64, 64, dtype=torch.bfloat16).cuda()
    k = torch.randn(1, 1, 128, 64, dtype=torch.bfloat16).cuda()
    with pytest.raises(DltError):
        _fa().attention(q, k, k, True, 1.0)  # causal needs Lq == Lk
    with pytest.raises(AssertionError):
        _fa().attention(q, k[..., :32], k, False, 1.0)


def test_gradients_that_cancel_stay_zero_with_fp32_inputs():
    """A query that sees a single key has p = 1 and dS = dP - delta = 0, so dq = dk = 0.  fp32 operands of the second
    products are rounded to bf16 on load: delta is formed from the same rounded dO as dP, or the difference of the two
    roundings (about 1e-1 at head dim 256) would show up as a gradient; and the backward kernels recompute the scores from
    the same hi + lo pairs as the forward kernel, so p is 1 and not exp of a rounding difference."""
    fa = _fa()
    q, k, v, do = orc.make_qkv(31, 2, 2, 200, 1, 120, 256, torch.float32)
    qg, kg, vg = (t.cuda().requires_grad_(True) for t in (q, k, v))
    o = fa.attention(qg, kg, vg, False, 0.3)
    o.backward(do.cuda())
    assert qg.grad.abs().max().item() <= 1e-4 and kg.grad.abs().max().item() <= 1e-3
    want = do.bfloat16().float().sum(dim=2, keepdim=True)        # dv = sum over the queries of the rounded dO
    assert (vg.grad.cpu() - want).abs().max().item() <= 1e-3 * want.abs().max().item()
