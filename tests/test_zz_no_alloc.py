"""dlt_swa_bwd_noalloc (the backward entry point that allocates nothing: delta lives in a static device array
inside the library) against dlt_swa_bwd with a caller-provided delta, through the C ABI: dq, dk, dv bit-equal,
on two calls in a row, the second on a smaller input (the shared scratch still holds the first call's values).
"""
import math

import pytest
import torch

from oracle import attn_oracle as orc

pytestmark = pytest.mark.gpu


def _call(noalloc, q, k, v, o, lse, do, shape, rope=None):
    from dl_templates_amd import _lib
    lib, P, S = _lib.load(), _lib.ptr, _lib.strides
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    desc, keep = (None, None) if rope is None else _lib.rope_desc(*rope, like=q, n_tokens=q.shape[2])
    head = (P(q), S(q), P(k), S(k), P(v), S(v), P(o), S(o), P(do), S(do))
    tail = (P(dq), S(dq), P(dk), S(dk), P(dv), S(dv), shape, desc, _lib.stream_of(q))
    if noalloc:
        rc = lib.dlt_swa_bwd_noalloc(*head, P(lse), S(lse), *tail)
    else:
        delta = torch.empty_like(lse)
        rc = lib.dlt_swa_bwd(*head, P(lse), P(delta), S(lse), *tail)
    _lib.check(rc)
    del keep
    return dq, dk, dv


def _case(seed, B, H, S, th, tw, W, d, dtype, with_rope=False):
    from dl_templates_amd import tiled_swa as sw
    N = th * tw * S
    q, k, v, do = (t.cuda() for t in orc.make_qkv(seed, B, H, N, N, d, d, dtype))
    scale = 1 / math.sqrt(d)
    rope = None
    if with_rope:
        rope = (orc.make_rope_idx(seed, th, tw, 0.1).cuda(), orc.rope_tables(8, th).cuda(), orc.rope_tables(8, tw).cuda())
    shape = sw._shape(q, k, v, S, th, tw, W, W, scale)
    o, lse = sw._forward(q, k, v, shape, rope)
    want = _call(False, q, k, v, o, lse, do, shape, rope)
    got = _call(True, q, k, v, o, lse, do, shape, rope)
    for name, a, b in zip(("dq", "dk", "dv"), got, want):
        assert torch.equal(a, b), f"{name} differs from dlt_swa_bwd"
    # and against the oracle, to the bar of the other backward tests
    if N <= 4096:
        qf, kf, vf, dof = (t.float().cpu() for t in (q, k, v, do))
        if with_rope:
            ref = orc.rope_swa_grads(qf, kf, vf, dof, rope[0].cpu(), rope[1].cpu(), rope[2].cpu(), S, th, tw, W, W, scale)
        else:
            ref = orc.tiled_swa_grads(qf, kf, vf, dof, S, th, tw, W, W, scale)
        for a, w in zip(got, ref[1:]):
            assert ((a.float().cpu() - w).abs().max() / w.abs().max().clamp_min(1e-3)).item() <= 5e-2


def test_two_calls_in_a_row_second_one_smaller():
    _case(1, 2, 8, 1, 64, 64, 6, 64, torch.bfloat16)          # config 3 shape: token-grid kernels, 65 536 delta values
    _case(2, 1, 2, 1, 20, 28, 3, 64, torch.bfloat16)          # smaller: most of the scratch keeps the first call's values
    _case(3, 1, 2, 16, 4, 5, 1, 32, torch.float16)            # tiles of 16 tokens: flash-family kernels
    _case(4, 1, 3, 3, 5, 4, 2, 32, torch.float32)             # generic kernels with the separate delta pre-pass
    _case(5, 1, 2, 1, 12, 20, 3, 64, torch.bfloat16, True)    # fused rotation


def test_sizes_beyond_the_scratch_are_rejected_before_any_launch():
    from dl_templates_amd import _lib, tiled_swa as sw
    lib, P, S = _lib.load(), _lib.ptr, _lib.strides
    B, H, th, tw, d = 1, 1, 8, 8, 32
    q = torch.zeros((B, H, th * tw, d), dtype=torch.bfloat16, device="cuda")
    lse = torch.zeros((B, H, th * tw), dtype=torch.float32, device="cuda")
    shape = sw._shape(q, q, q, 1, th, tw, 1, 1, 1.0)
    big = (_lib.c_int64 * 3)(0, 0, _lib.NOALLOC_MAX_DELTA // (th * tw - 1) + 1)    # last token lands beyond the scratch
    rc = lib.dlt_swa_bwd_noalloc(P(q), S(q), P(q), S(q), P(q), S(q), P(q), S(q), P(q), S(q), P(lse), big,
                                 P(q), S(q), P(q), S(q), P(q), S(q), shape, None, _lib.stream_of(q))
    assert rc == 1 and b"scratch" in lib.dlt_last_error()
    neg = (_lib.c_int64 * 3)(0, 0, -1)
    rc = lib.dlt_swa_bwd_noalloc(P(q), S(q), P(q), S(q), P(q), S(q), P(q), S(q), P(q), S(q), P(lse), neg,
                                 P(q), S(q), P(q), S(q), P(q), S(q), shape, None, _lib.stream_of(q))
    assert rc == 1 and b"negative" in lib.dlt_last_error()
    # exactly at the limit (1 Mi tokens) is accepted by the size check: B * H * N = 2^20 (checked without launching: NULL q)
    shape = _lib.SwaShape(1, 16, 1, 256, 256, 1, 1, 32, 32, 1.0, 0)
    st = (_lib.c_int64 * 3)(16 * 65536, 65536, 1)
    rc = lib.dlt_swa_bwd_noalloc(None, S(q), P(q), S(q), P(q), S(q), P(q), S(q), P(q), S(q), P(lse), st,
                                 P(q), S(q), P(q), S(q), P(q), S(q), shape, None, _lib.stream_of(q))
    assert rc == 1 and b"NULL" in lib.dlt_last_error()


def _prepared(seed, B, H, th, tw, W, d):
    from dl_templates_amd import tiled_swa as sw
    N = th * tw
    q, k, v, do = (t.cuda() for t in orc.make_qkv(seed, B, H, N, N, d, d, torch.bfloat16))
    shape = sw._shape(q, k, v, 1, th, tw, W, W, 1 / math.sqrt(d))
    o, lse = sw._forward(q, k, v, shape, None)
    return q, k, v, o, lse, do, shape


def _launch_noalloc(args, outs):
    from dl_templates_amd import _lib
    lib, P, S = _lib.load(), _lib.ptr, _lib.strides
    q, k, v, o, lse, do, shape = args
    dq, dk, dv = outs
    _lib.check(lib.dlt_swa_bwd_noalloc(P(q), S(q), P(k), S(k), P(v), S(v), P(o), S(o), P(do), S(do), P(lse), S(lse),
                                       P(dq), S(dq), P(dk), S(dk), P(dv), S(dv), shape, None, _lib.stream_of(q)))


def test_a_warm_call_leaves_device_memory_as_it_was():
    """After one call outside any capture (which resolves the scratch symbol and sets the kernels' LDS attribute once
    per device), a further call changes neither the free device memory the driver reports nor torch's allocator."""
    args = _prepared(7, 1, 4, 32, 32, 6, 64)
    outs = tuple(torch.empty_like(t) for t in args[:3])
    _launch_noalloc(args, outs)   # warm
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    alloc0, reserved0 = torch.cuda.memory_allocated(), torch.cuda.memory_reserved()
    for _ in range(3):
        _launch_noalloc(args, outs)
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0, (free0, free1)
    assert (torch.cuda.memory_allocated(), torch.cuda.memory_reserved()) == (alloc0, reserved0)


def test_captured_in_a_hip_graph_every_replay_equals_the_eager_call():
    """The call it is meant for: recorded into a HIP graph (after a warm call outside the capture) and replayed, with
    eager work and synchronisations between the replays; every replay must reproduce the eager gradients bit for bit."""
    args = _prepared(8, 2, 4, 32, 48, 6, 64)
    want = tuple(torch.empty_like(t) for t in args[:3])
    _launch_noalloc(args, want)   # warm call, outside the capture; also the eager result
    torch.cuda.synchronize()
    outs = tuple(torch.empty_like(t) for t in args[:3])
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            _launch_noalloc(args, outs)
    torch.cuda.current_stream().wait_stream(side)
    small = _prepared(9, 1, 2, 16, 16, 3, 64)
    for rep in range(4):
        for t in outs:
            t.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        for name, a, b in zip(("dq", "dk", "dv"), outs, want):
            assert torch.equal(a, b), f"replay {rep}: {name} differs from the eager call"
        # eager work on the same scratch between the replays (a smaller call overwrites the head of it)
        _launch_noalloc(small, tuple(torch.empty_like(t) for t in small[:3]))
        torch.cuda.synchronize()
