"""Host-side checks that need no GPU: the C-ABI library loads, exports every symbol that
include/dlt.h declares, and rejects bad arguments before launching anything."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _lib():
    from dl_templates_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("libdlt_hip.so not built (run __graft_entry__.build())")
    return _lib


def test_library_exports_every_declared_symbol():
    L = _lib()
    lib = L.load()
    header = open(os.path.join(ROOT, "include", "dlt.h")).read()
    declared = set(re.findall(r"\b(dlt_[a-z0-9_]+)\s*\(", header))
    declared -= {"dlt_dtype_t"}
    assert declared, "no declarations found in include/dlt.h"
    for name in sorted(declared):
        assert hasattr(lib, name), f"{name} is declared in dlt.h but not exported"
    assert set(L.EXPORTS) == declared
    assert lib.dlt_version() >= 1


def test_argument_validation_happens_before_any_launch():
    L = _lib()
    lib = L.load()
    shape = L.SwaShape(1, 1, 1, 4, 4, 1, 1, 64, 64, 1.0, 7)  # bad dtype
    st4 = (ctypes.c_int64 * 4)(1, 1, 1, 1)
    st3 = (ctypes.c_int64 * 3)(1, 1, 1)
    one = ctypes.c_void_p(16)
    rc = lib.dlt_swa_fwd(one, st4, one, st4, one, st4, one, st4, one, st3, shape, None, None)
    assert rc == 1 and b"dtype" in lib.dlt_last_error()
    shape = L.SwaShape(1, 1, 1, 4, 4, 1, 1, 64, 64, 1.0, 0)
    rc = lib.dlt_swa_fwd(None, st4, one, st4, one, st4, one, st4, one, st3, shape, None, None)
    assert rc == 1 and b"NULL" in lib.dlt_last_error()
    shape = L.SwaShape(1, 1, 1, 4, 4, 1, 1, 512, 64, 1.0, 0)
    rc = lib.dlt_swa_fwd(one, st4, one, st4, one, st4, one, st4, one, st3, shape, None, None)
    assert rc == 2 and b"head dims" in lib.dlt_last_error()
    shape = L.SwaShape(1, 1, 1, 4, 4, 1, 1, 64, 64, float("inf"), 0)
    rc = lib.dlt_swa_fwd(one, st4, one, st4, one, st4, one, st4, one, st3, shape, None, None)
    assert rc == 1 and b"sm_scale" in lib.dlt_last_error()
    rc = lib.dlt_flash_fwd(one, st4, one, st4, one, st4, one, st4, one, st3, L.FlashShape(1, 1, 8, 8, 64, 64, float("nan"), 0, 0), None)
    assert rc == 1 and b"sm_scale" in lib.dlt_last_error()
    st5 = (ctypes.c_int64 * 5)(1, 1, 1, 1, 1)
    shape = L.SwaShape(1, 1, 6, 4, 4, 1, 1, 64, 64, 1.0, 0)  # tile of 2 x 2 pixels is not 6 tokens
    rc = lib.dlt_swa_fwd_image(one, st5, one, st5, one, st5, one, st5, one, st3, shape, L.SwaTile(2, 2), None, None)
    assert rc == 1 and b"b_size" in lib.dlt_last_error()
    rc = lib.dlt_swa_image_offsets(0, 4, 2, 2, 8, 1, one, None)
    assert rc == 1 and b"grid" in lib.dlt_last_error()
    fshape = L.FlashShape(1, 1, 8, 16, 64, 64, 1.0, 1, 0)  # causal with Lq != Lk
    rc = lib.dlt_flash_fwd(one, st4, one, st4, one, st4, one, st4, one, st3, fshape, None)
    assert rc == 1 and b"causal" in lib.dlt_last_error()
    rope = L.RopeDesc(16, 16, 16, 16, 16, 8, 4, 4)
    rc = lib.dlt_rope2d(one, st3, 1, 4, 16, rope, 0, 0, None)  # 4R = 32 > C = 16
    assert rc == 1 and b"n_rdim" in lib.dlt_last_error()
    assert lib.dlt_rope2d(None, st3, 0, 0, 16, L.RopeDesc(0, 0, 0, 0, 0, 0, 0, 0), 0, 0, None) == 0


def test_product_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "dl_templates_amd")
    for fn in os.listdir(pkg):
        if fn.endswith(".py"):
            src = open(os.path.join(pkg, fn)).read()
            assert "oracle" not in src, f"{fn} must not reference the oracle"


def test_table_context_matches_oracle_tables():
    import torch
    from dl_templates_amd.rope2d import FusedRotaryPositionEncodingContext as Ctx
    from dl_templates_amd.fused_rope2d import FusedInplaceRotaryPositionEncoding2D as M
    from oracle import attn_oracle as orc
    assert (Ctx(16, 64).cs_components - orc.rope_tables(8, 64)).abs().max().item() <= 1.2e-7
    assert torch.equal(M.encode_idx(5, 7), orc.encode_idx(5, 7))
    m = M(32, 8, 9)
    assert m.row_buffer.cs_components.shape == (8, 8, 2) and m.col_buffer.cs_components.shape == (9, 8, 2)


def test_rope_operands_on_the_host_raise_before_any_launch():
    """idx / tables are dereferenced by the kernels: the attention wrappers must refuse host tensors (what
    encode_idx returns without a default device) instead of handing a host pointer to the GPU."""
    import pytest
    import torch
    from dl_templates_amd import _lib
    from dl_templates_amd.fused_rope2d import FusedInplaceRotaryPositionEncoding2D as M

    class OnGpu:   # stands in for the CUDA tensor the rotation is applied to (no GPU in the CPU suite)
        is_cuda = True
        device = torch.device("cuda:0")

    idx = M.encode_idx(4, 4)
    tab = torch.zeros(4, 8, 2)
    with pytest.raises(RuntimeError, match="ROCm GPU only"):
        _lib.rope_desc(idx, tab, tab, like=OnGpu())
    with pytest.raises(ValueError, match="entries for"):
        _lib.rope_desc(idx, tab, tab, n_tokens=17)
    with pytest.raises(TypeError):
        _lib.rope_desc(idx.long(), tab, tab)
