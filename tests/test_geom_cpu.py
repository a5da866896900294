"""CPU checks of the geometry header the host code, the debug exports and every kernel share
(dl_templates_amd/csrc/dlt_geom.h): window ranges against the oracle's neighbour masks
(src/tiled_swa.py:701-713), the idx decode (src/fused_rope2d.py:40-45), the token -> pixel map of the
image layout (src/tiled_swa.py:753-755) and the exact multiply-shift division it uses.  The header is
compiled with the host compiler through tests/geom_shim.cpp; no GPU is involved."""
import ctypes
import os
import random
import shutil
import subprocess

import numpy as np
import pytest

from oracle import attn_oracle as orc

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(scope="module")
def shim(tmp_path_factory):
    cxx = shutil.which("g++") or shutil.which("c++")
    if cxx is None:
        pytest.skip("no host C++ compiler")
    out = str(tmp_path_factory.mktemp("geom") / "libgeom_shim.so")
    subprocess.run([cxx, "-O1", "-std=c++17", "-shared", "-fPIC", os.path.join(HERE, "geom_shim.cpp"), "-o", out], check=True)
    lib = ctypes.CDLL(out)
    lib.shim_fastdiv.restype = ctypes.c_uint
    lib.shim_fastdiv.argtypes = [ctypes.c_uint, ctypes.c_uint]
    return lib


def test_fastdiv_is_exact_below_2_pow_31(shim):
    rng = random.Random(0)
    divisors = [1, 2, 3, 5, 7, 16, 17, 48, 63, 64, 65, 100, 4095, 4096, 4097, 65535, 65537, 1000003, (1 << 30) - 1, 1 << 30,
                (1 << 31) - 1] + [rng.randrange(1, 1 << rng.randrange(1, 31)) for _ in range(200)]
    for d in divisors:
        edge = [0, 1, d - 1, d, d + 1, 2 * d - 1, 2 * d, (1 << 31) - 1, ((1 << 31) - 1) // d * d, ((1 << 31) - 1) // d * d - 1]
        for n in edge + [rng.randrange(0, 1 << 31) for _ in range(50)]:
            n = max(0, min(n, (1 << 31) - 1))
            assert shim.shim_fastdiv(n, d) == n // d, (n, d)


@pytest.mark.parametrize("th,tw,bh,bw", [(2, 3, 4, 4), (3, 2, 2, 5), (4, 5, 1, 1), (1, 4, 3, 1), (5, 1, 1, 7), (16, 16, 4, 4), (7, 9, 6, 8)])
def test_token_pixel_map_matches_the_oracle(shim, th, tw, bh, bw):
    index = orc.image_token_index(th, tw, bh, bw)              # [IH, IW] -> token
    y, x = ctypes.c_uint(), ctypes.c_uint()
    for n in range(th * tw * bh * bw):
        shim.shim_token_pixel(bh, bw, tw, n, ctypes.byref(y), ctypes.byref(x))
        assert index[y.value, x.value] == n
    i = ctypes.c_uint()
    S = bh * bw
    for xs in range(tw * S):                                    # slot inside one grid row
        shim.shim_slot_pixel(bh, bw, tw, xs, ctypes.byref(i), ctypes.byref(x))
        assert index[i.value, x.value] == xs                    # grid row 0: token == slot


def test_window_ranges_match_the_neighbour_masks(shim):
    out = (ctypes.c_int * 8)()
    rng = random.Random(1)
    for _ in range(60):
        th, tw, S = rng.randint(1, 6), rng.randint(1, 7), rng.choice([1, 1, 2, 16])
        WR, WC = rng.randint(0, 4), rng.randint(0, 4)
        mask = orc.neighbor_mask(th, tw, WR, WC)
        XL = tw * S
        for r in range(th):
            for c in range(tw):
                x = c * S + rng.randrange(S)
                shim.shim_key_range(0, th, tw, S, min(WR, th), min(WC, tw), XL, XL, r, x, out)
                got = np.zeros((th, tw), dtype=bool)
                assert out[2] % S == 0 and out[3] % S == 0
                got[out[0]:out[1] + 1, out[2] // S:out[3] // S] = True
                assert np.array_equal(got.reshape(-1), mask[r * tw + c])
                assert list(out[4:8]) == list(out[0:4])      # the window is symmetric: queries of a key == keys of a query


def test_dense_and_causal_ranges(shim):
    out = (ctypes.c_int * 8)()
    shim.shim_key_range(1, 1, 1, 1, 0, 0, 50, 70, 0, 13, out)     # dense: every key, every query
    assert list(out) == [0, 0, 0, 70, 0, 0, 0, 50]
    shim.shim_key_range(2, 1, 1, 1, 0, 0, 64, 64, 0, 13, out)     # causal: keys 0..13, queries 13..63
    assert list(out) == [0, 0, 0, 14, 0, 0, 13, 64]


def test_idx_decode_matches_the_oracle(shim):
    vals = [-1, 0, 0xFFFF, 0x7FFF0000 | 5, (3 << 16) | 0xFFFF, (0x8000 << 16) | 7, (12 << 16) | 34, -65536, 65535]
    vals = [v - (1 << 32) if v >= (1 << 31) else v for v in vals]
    rows, cols = orc.decode_idx(np.array(vals, dtype=np.int32))
    for v, r, c in zip(vals, rows, cols):
        assert shim.shim_rope_row(v) == r and shim.shim_rope_col(v) == c
