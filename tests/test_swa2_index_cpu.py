"""Host model of the streaming token-grid kernels' staging and operand-read maps (tests/swa2_shim.cpp over
dl_templates_amd/csrc/swa2_index.h, the header the kernels compute every global and LDS offset with): for every workgroup,
chunk, wave, lane and copy instruction of a problem it checks that global reads stay inside the tensor, LDS writes and
reads stay inside the bytes the launcher asks for and inside their own region, that every operand read finds the token
and head dims the matrix layout expects, and that the window test equals the shared geometry routine (the neighbour sets
of src/tiled_swa.py:86-104,701-713): every key of a window visible exactly once over the column passes.  Classes: head dim
64 with 4 / 6 / 8 / 10 column groups, head dim 128 with 4 / 6; windows wider than a class in 2 to 4 column passes (the
product instantiates 4 and 6 and walks wider windows in passes).  No GPU is involved."""
import ctypes
import os
import shutil
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(scope="module")
def shim(tmp_path_factory):
    cxx = shutil.which("g++") or shutil.which("c++")
    if cxx is None:
        pytest.skip("no host C++ compiler")
    out = str(tmp_path_factory.mktemp("swa2") / "libswa2_shim.so")
    subprocess.run([cxx, "-O2", "-std=c++17", "-Wno-unknown-pragmas", "-shared", "-fPIC", os.path.join(HERE, "swa2_shim.cpp"), "-o", out],
                   check=True)
    lib = ctypes.CDLL(out)
    lib.swa2_model.argtypes = [ctypes.c_int] * 11 + [ctypes.c_longlong] * 2 + [ctypes.c_int] * 2
    lib.swa2_model_message.restype = ctypes.c_char_p
    return lib


ALL = [(64, 4), (64, 6), (64, 8), (64, 10), (128, 4), (128, 6)]


def _classes(WC):
    """(head dim, column groups, column passes) of every class, with the fewest passes that hold a window of 2 WC + 1
    columns (at most 4)."""
    need = (4 + 2 * WC + 3) // 4
    return [(d, n, -(-need // n)) for d, n in ALL if -(-need // n) <= 4]


def _run(shim, D, NCG, npass, TR, TC, WR, WC, pad=0, ls2=1, S=1, band=8):
    """TC, WC in tiles of S tokens; band: grid rows per workgroup (16: two stacked patches per wave)."""
    sn2 = 2 * D + pad
    slab = (TR * TC * S - 1) * sn2 + 2 * D
    scal = (TR * TC * S - 1) * ls2 + 1
    rc = shim.swa2_model(D, NCG, npass, band, TR, TC, WR, WC, S, sn2, ls2, slab, scal, shim.swa2_class_lds(D, NCG, 0), shim.swa2_class_lds(D, NCG, 1))
    assert rc == 0, f"D={D} NCG={NCG} x {npass} band {band} grid {TR}x{TC} tiles of {S} window ({WR},{WC}) stride {sn2}: {shim.swa2_model_message().decode()}"


# grids of the GPU tests (ragged, one token, narrower than a band, windows wider than the grid) and of the benchmark
GRIDS = [(1, 1), (1, 7), (5, 1), (3, 5), (8, 16), (9, 17), (13, 29), (16, 16), (20, 28), (33, 18), (17, 47), (40, 40)]
WINDOWS = [(0, 0), (1, 1), (3, 3), (6, 6), (2, 6), (7, 7), (10, 10), (1, 10), (12, 3), (11, 11), (14, 14), (3, 14), (15, 15), (18, 18), (9, 18), (30, 18),
           (5, 22), (11, 29), (2, 34), (8, 46)]


@pytest.mark.parametrize("TR,TC", GRIDS)
def test_every_class_on_small_and_ragged_grids(shim, TR, TC):
    for WR, WC in WINDOWS:
        for D, NCG, npass in _classes(WC):
            _run(shim, D, NCG, npass, TR, TC, WR, WC)
            if D == 128:   # the forward kernel with two stacked patches per wave: bands of 16 rows
                _run(shim, D, NCG, npass, TR, TC, WR, WC, band=16)


def test_more_passes_than_needed_change_nothing(shim):
    # a pass whose column groups all lie beyond the window sees no key
    _run(shim, 64, 4, 3, 20, 28, 3, 5)
    _run(shim, 128, 6, 2, 17, 47, 6, 2)


def test_benchmark_grids_and_strided_rows(shim):
    for band in (8, 16):
        _run(shim, 128, 6, 1, 128, 128, 10, 10, band=band)
        _run(shim, 128, 6, 1, 96, 160, 10, 10, band=band)
        _run(shim, 128, 6, 4, 128, 128, 20, 46, band=band)
        _run(shim, 128, 4, 2, 21, 37, 5, 11, pad=768, ls2=3, band=band)
    _run(shim, 64, 4, 1, 64, 64, 6, 6)
    for D, NCG, npass, WC in [(64, 8, 1, 11), (64, 8, 1, 14), (64, 10, 1, 15), (64, 10, 1, 18), (128, 4, 2, 11), (128, 6, 2, 18),
                              (64, 6, 3, 34), (128, 6, 4, 46)]:
        _run(shim, D, NCG, npass, 128, 128, min(WC, 20), WC)
        _run(shim, D, NCG, npass, 96, 160, min(WC, 20), WC)
    # token rows that are strided views of a packed projection, scalars with a stride
    for D, NCG, npass, WC in [(64, 4, 1, 3), (64, 10, 1, 16), (128, 6, 1, 9), (128, 4, 2, 11), (64, 6, 2, 17)]:
        _run(shim, D, NCG, npass, 21, 37, 5, WC, pad=6 * D, ls2=3)


@pytest.mark.parametrize("S", [2, 3, 4, 8, 9, 15])
def test_tiles_of_fewer_than_16_tokens(shim, S):
    """A token sees whole tiles: S WC + (x mod S) slots to its left, S WC + S - 1 - (x mod S) to its right."""
    for TR, TC, WR, WC in [(5, 7, 1, 1), (9, 3, 2, 0), (3, 11, 0, 2), (10, 6, 3, 1), (1, 1, 0, 0)]:
        need = (4 + 2 * (S * WC + S - 1) + 3) // 4
        for D, NCG in [(64, 4), (64, 6), (128, 4), (128, 6)]:
            npass = -(-need // NCG)
            if npass <= 4:
                _run(shim, D, NCG, npass, TR, TC, WR, WC, S=S)
                if D == 128:
                    _run(shim, D, NCG, npass, TR, TC, WR, WC, S=S, band=16)


def test_the_model_notices_a_wrong_launch(shim):
    # a window wider than class x passes, and an LDS size below what the class needs
    rc = shim.swa2_model(64, 4, 1, 8, 16, 16, 3, 7, 1, 128, 1, 16 * 16 * 128, 256, shim.swa2_class_lds(64, 4, 0), shim.swa2_class_lds(64, 4, 1))
    assert rc == 1 and b"column groups" in shim.swa2_model_message()
    rc = shim.swa2_model(64, 6, 1, 8, 16, 16, 3, 7, 1, 128, 1, 16 * 16 * 128, 256, shim.swa2_class_lds(64, 4, 0), shim.swa2_class_lds(64, 6, 1))
    assert rc == 1 and b"LDS" in shim.swa2_model_message()
    # a slab one row short: the last row's copy must be caught
    rc = shim.swa2_model(64, 4, 1, 8, 16, 16, 3, 3, 1, 128, 1, 16 * 16 * 128 - 128, 256, shim.swa2_class_lds(64, 4, 0), shim.swa2_class_lds(64, 4, 1))
    assert rc == 1 and b"global" in shim.swa2_model_message()
