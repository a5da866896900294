"""Which kernel family a call is routed to, asked through the C ABI without a GPU: under dlt_dry_run(1) the entry points
validate and route but launch nothing, and dlt_last_kernel_family() names the family.  The cases pin the routing table
that include/dlt.h documents, so that a call landing on the (several times slower) generic kernels is visible to a C
caller: head dims outside the tuned shapes, windows wider than 93 columns, rows that are not 16-byte aligned, fp32."""
import ctypes
import os

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BF16, FP16, FP32 = 0, 1, 2


@pytest.fixture(scope="module")
def L():
    from dl_templates_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("libdlt_hip.so not built (run __graft_entry__.build())")
    lib = _lib.load()
    lib.dlt_dry_run(1)
    yield _lib
    lib.dlt_dry_run(0)


def _contig(B, H, N, D, pad=0):
    row = D + pad
    return (ctypes.c_int64 * 4)(H * N * row, N * row, row, 1)


def _swa(L, S, th, tw, WR, WC, dk, dv, dtype, backward=False, rope_R=0, align=256, pad=0, B=1, H=2, table_len=64, prerot=False):
    lib = L.load()
    N = S * th * tw
    ptr = ctypes.c_void_p(align)        # never dereferenced: only its alignment is looked at
    qs, vs = _contig(B, H, N, dk, pad), _contig(B, H, N, dv, pad)
    ls = (ctypes.c_int64 * 3)(H * N, N, 1)
    shape = L.SwaShape(B, H, S, th, tw, WR, WC, dk, dv, 0.125, dtype)
    rope = L.RopeDesc(256, 256, 256, 2 * rope_R, 2 * rope_R, rope_R, table_len, table_len) if rope_R else None
    if not backward:
        if prerot:
            rc = lib.dlt_swa_fwd_rot(ptr, qs, ptr, qs, ptr, vs, ptr, vs, ptr, ls, ctypes.c_void_p(align * 3), qs, ctypes.c_void_p(align * 5), qs, shape, rope, None)
        else:
            rc = lib.dlt_swa_fwd(ptr, qs, ptr, qs, ptr, vs, ptr, vs, ptr, ls, shape, rope, None)
    else:
        fn = lib.dlt_swa_bwd_rot if prerot else lib.dlt_swa_bwd
        rc = fn(ptr, qs, ptr, qs, ptr, vs, ptr, vs, ptr, vs, ptr, ptr, ls, ptr, qs, ptr, qs, ptr, vs, shape, rope, None)
    assert rc == 0, lib.dlt_last_error()
    return L.KERNEL_FAMILIES[lib.dlt_last_kernel_family()]


def _flash(L, Lq, Lk, dk, dv, dtype, causal=False, backward=False, align=256, pad=0, B=1, H=2):
    lib = L.load()
    ptr = ctypes.c_void_p(align)
    qs, ks, vs, os_ = _contig(B, H, Lq, dk, pad), _contig(B, H, Lk, dk, pad), _contig(B, H, Lk, dv, pad), _contig(B, H, Lq, dv, pad)
    ls = (ctypes.c_int64 * 3)(H * Lq, Lq, 1)
    shape = L.FlashShape(B, H, Lq, Lk, dk, dv, 0.125, int(causal), dtype)
    if not backward:
        rc = lib.dlt_flash_fwd(ptr, qs, ptr, ks, ptr, vs, ptr, os_, ptr, ls, shape, None)
    else:
        rc = lib.dlt_flash_bwd(ptr, qs, ptr, ks, ptr, vs, ptr, os_, ptr, os_, ptr, ptr, ls, ptr, qs, ptr, ks, ptr, vs, shape, None)
    assert rc == 0, lib.dlt_last_error()
    return L.KERNEL_FAMILIES[lib.dlt_last_kernel_family()]


@pytest.mark.parametrize("backward", [False, True])
def test_token_grid_routing_table(L, backward):
    kw = dict(backward=backward)
    # the benchmark configurations
    assert _swa(L, 1, 64, 64, 6, 6, 64, 64, BF16, **kw) == "marching"                      # config 3 without rotation
    assert _swa(L, 1, 64, 64, 6, 6, 64, 64, BF16, rope_R=8, prerot=True, **kw) == "marching"   # config 3, rotated q / k kept
    assert _swa(L, 1, 128, 128, 10, 10, 128, 128, BF16, **kw) == "streaming"               # config 4
    assert _swa(L, 1, 96, 160, 10, 10, 128, 128, FP16, **kw) == "streaming"
    # head dim 64 beyond the marching kernels' 13 x 13 window, head dims in multiples of 32 below a class
    assert _swa(L, 1, 40, 40, 9, 9, 64, 64, BF16, **kw) == "streaming"
    # windows wider than 21 columns: the streaming kernels in column passes (any number of rows)
    assert _swa(L, 1, 40, 40, 11, 11, 64, 64, BF16, **kw) == "streaming"
    assert _swa(L, 1, 40, 90, 30, 34, 128, 128, FP16, **kw) == "streaming"
    assert _swa(L, 1, 40, 40, 3, 3, 96, 96, BF16, **kw) == "tile"
    assert _swa(L, 1, 40, 40, 3, 3, 32, 64, BF16, **kw) == "tile"
    # rotation inside the tile loads (nothing kept), rotation at head dim 128 or with 16 rotary pairs
    assert _swa(L, 1, 40, 40, 3, 3, 64, 64, BF16, rope_R=8, **kw) == ("marching" if not backward else "tile")
    assert _swa(L, 1, 40, 40, 3, 3, 128, 128, BF16, rope_R=16, prerot=True, **kw) == "tile"
    # what falls to the generic kernels: head dims that are not multiples of 32 or straddle the classes, windows of more
    # than 93 columns (or wide ones below a class's head dim, or with rotation), fp32, rows that are not 16-byte
    # aligned, tiles that are neither multiples of 16 tokens nor 2 ... 15 tokens at head dim 64 / 128
    assert _swa(L, 1, 40, 40, 3, 3, 80, 80, BF16, **kw) == "generic"
    assert _swa(L, 1, 40, 40, 3, 3, 64, 128, BF16, **kw) == "generic"
    assert _swa(L, 1, 8, 200, 3, 47, 64, 64, BF16, **kw) == "generic"                     # 95 columns: more than 4 passes of 6 groups
    assert _swa(L, 1, 40, 40, 11, 11, 96, 96, BF16, **kw) == "generic"                    # wide window below the class's head dim
    assert _swa(L, 1, 40, 40, 3, 11, 64, 64, BF16, rope_R=8, **kw) == "generic"           # wide window with rotation
    assert _swa(L, 1, 40, 40, 3, 3, 64, 64, FP32, **kw) == "generic"
    assert _swa(L, 1, 40, 40, 3, 3, 64, 64, BF16, align=2, **kw) == "generic"
    assert _swa(L, 1, 40, 40, 3, 3, 64, 64, BF16, pad=1, **kw) == "generic"
    assert _swa(L, 9, 8, 8, 1, 1, 32, 32, BF16, **kw) == "generic"
    assert _swa(L, 24, 8, 8, 1, 1, 64, 64, BF16, **kw) == "generic"
    # tiles of 2 ... 15 tokens at head dim 64 / 128: the streaming kernels on the grid of token slots
    assert _swa(L, 9, 8, 8, 1, 1, 64, 64, BF16, **kw) == "streaming"
    assert _swa(L, 4, 32, 32, 2, 2, 128, 128, FP16, **kw) == "streaming"
    # tiles of 16 k tokens: the flash family in tile mode (its kernels pad head dims inside)
    assert _swa(L, 16, 16, 16, 1, 1, 32, 32, FP16, **kw) == "flash"
    assert _swa(L, 64, 16, 16, 1, 1, 64, 64, BF16, **kw) == "flash"
    assert _swa(L, 16, 8, 8, 1, 1, 40, 72, BF16, **kw) == "flash"


@pytest.mark.parametrize("backward", [False, True])
def test_flash_routing_table(L, backward):
    kw = dict(backward=backward)
    assert _flash(L, 4096, 8192, 64, 128, BF16, **kw) == "flash"                           # config 5
    assert _flash(L, 4096, 4096, 64, 64, FP16, causal=True, **kw) == "flash"
    assert _flash(L, 1000, 777, 40, 96, BF16, **kw) == "flash"                             # multiples of 8
    assert _flash(L, 512, 512, 100, 100, BF16, **kw) == "generic"                          # rows of 200 bytes
    assert _flash(L, 512, 512, 136, 136, BF16, **kw) == "generic"                          # above 128
    assert _flash(L, 512, 512, 64, 64, FP32, **kw) == "generic"
    assert _flash(L, 512, 512, 64, 64, BF16, align=4, **kw) == "generic"


def test_dry_run_is_per_thread_and_off_by_default(L):
    import threading
    lib = L.load()
    seen = {}

    def other():
        # a fresh thread is not in dry-run mode: a NULL pointer is still refused before anything else happens
        seen["family"] = lib.dlt_last_kernel_family()
    t = threading.Thread(target=other)
    t.start()
    t.join()
    assert seen["family"] == 0
    assert _swa(L, 1, 16, 16, 3, 3, 64, 64, BF16) == "marching"
    assert lib.dlt_last_kernel_family() == 1
