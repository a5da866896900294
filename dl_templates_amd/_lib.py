"""ctypes binding of ``libdlt_hip.so`` (declared in ``include/dlt.h``).

The shared object is built in-tree by ``dl_templates_amd/csrc/Makefile`` (see
``__graft_entry__.build``).  It is loaded after ``import torch`` so that it binds to the
HIP runtime PyTorch already holds: one runtime per process, shared streams and pointers.
There is no CPU fallback: a missing library or a failing call raises.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
import threading
from ctypes import POINTER, Structure, c_char_p, c_float, c_int, c_int32, c_int64, c_void_p

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libdlt_hip.so")
CSRC_DIR = os.path.join(_HERE, "csrc")

DLT_BF16, DLT_FP16, DLT_FP32 = 0, 1, 2
_DTYPES = {torch.bfloat16: DLT_BF16, torch.float16: DLT_FP16, torch.float32: DLT_FP32}

EXPORTS = (
    "dlt_last_error", "dlt_version", "dlt_rope2d", "dlt_rope2d_pair", "dlt_rope_pe_mask",
    "dlt_swa_fwd", "dlt_swa_bwd", "dlt_swa_neighbors", "dlt_flash_fwd", "dlt_flash_bwd",
    "dlt_timing_enable", "dlt_timing_collect", "dlt_debug_copy",
    "dlt_swa_fwd_image", "dlt_swa_bwd_image", "dlt_swa_image_offsets", "dlt_swa_fwd_rot", "dlt_swa_bwd_rot",
    "dlt_swa_bwd_noalloc", "dlt_dry_run", "dlt_last_kernel_family",
)
KERNEL_FAMILIES = ("none", "marching", "streaming", "tile", "flash", "generic")   # DLT_FAMILY_* of include/dlt.h
NOALLOC_MAX_DELTA = 1 << 20  # DLT_NOALLOC_MAX_DELTA of include/dlt.h
KERNEL_NAMES = ("rope2d", "attn_fwd", "attn_delta", "attn_bwd_kv", "attn_bwd_q")


class DltError(RuntimeError):
    """A libdlt_hip entry point returned a non-zero status."""

    def __init__(self, code: int, message: str):
        super().__init__(f"libdlt_hip error {code}: {message}")
        self.code = code


class RopeDesc(Structure):
    _fields_ = [
        ("idx", c_void_p), ("row_cs", c_void_p), ("col_cs", c_void_p),
        ("row_cs_stride0", c_int64), ("col_cs_stride0", c_int64),
        ("n_rdim", c_int32), ("row_len", c_int32), ("col_len", c_int32),
    ]


class KernelTime(Structure):
    _fields_ = [("kernel", c_int32), ("ms", c_float)]


class SwaShape(Structure):
    _fields_ = [
        ("B", c_int32), ("H", c_int32), ("b_size", c_int32), ("t_height", c_int32), ("t_width", c_int32),
        ("row_size", c_int32), ("col_size", c_int32), ("dk", c_int32), ("dv", c_int32),
        ("sm_scale", c_float), ("dtype", c_int32),
    ]


class SwaTile(Structure):
    _fields_ = [("bh", c_int32), ("bw", c_int32)]


class FlashShape(Structure):
    _fields_ = [
        ("B", c_int32), ("H", c_int32), ("Lq", c_int32), ("Lk", c_int32), ("dk", c_int32), ("dv", c_int32),
        ("sm_scale", c_float), ("causal", c_int32), ("dtype", c_int32),
    ]


_lib = None
_lock = threading.Lock()


def build(verbose: bool = False) -> str:
    """Compile every HIP source for gfx950 into ``libdlt_hip.so`` (always recompiles)."""
    jobs = str(min(16, os.cpu_count() or 8))
    subprocess.run(["make", "-C", CSRC_DIR, "clean"], check=True, capture_output=not verbose)
    r = subprocess.run(["make", "-C", CSRC_DIR, "-j", jobs], capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("building libdlt_hip.so failed:\n" + r.stdout[-4000:] + r.stderr[-4000:])
    if verbose:
        print(r.stdout[-2000:])
    return LIB_PATH


def _declare(lib) -> None:
    P64 = POINTER(c_int64)
    lib.dlt_last_error.restype = c_char_p
    lib.dlt_last_error.argtypes = []
    lib.dlt_version.restype = c_int
    lib.dlt_rope2d.restype = c_int
    lib.dlt_rope2d.argtypes = [c_void_p, P64, c_int64, c_int64, c_int64, POINTER(RopeDesc), c_int, c_int, c_void_p]
    lib.dlt_rope2d_pair.restype = c_int
    lib.dlt_rope2d_pair.argtypes = [c_void_p, P64, c_int64, c_void_p, P64, c_int64, c_int64, c_int64,
                                    POINTER(RopeDesc), c_int, c_int, c_void_p]
    lib.dlt_rope_pe_mask.restype = c_int
    lib.dlt_rope_pe_mask.argtypes = [c_void_p, c_int64, c_void_p, c_void_p]
    lib.dlt_swa_neighbors.restype = c_int
    lib.dlt_swa_neighbors.argtypes = [c_int32, c_int32, c_int32, c_int32, c_void_p, c_void_p]
    fwd = [c_void_p, P64, c_void_p, P64, c_void_p, P64, c_void_p, P64, c_void_p, P64]
    bwd = [c_void_p, P64] * 5 + [c_void_p, c_void_p, P64] + [c_void_p, P64] * 3
    lib.dlt_swa_fwd.restype = c_int
    lib.dlt_swa_fwd.argtypes = fwd + [POINTER(SwaShape), POINTER(RopeDesc), c_void_p]
    lib.dlt_swa_bwd.restype = c_int
    lib.dlt_swa_bwd.argtypes = bwd + [POINTER(SwaShape), POINTER(RopeDesc), c_void_p]
    lib.dlt_swa_bwd_noalloc.restype = c_int
    lib.dlt_swa_bwd_noalloc.argtypes = [c_void_p, P64] * 5 + [c_void_p, P64] + [c_void_p, P64] * 3 + [
        POINTER(SwaShape), POINTER(RopeDesc), c_void_p]
    lib.dlt_swa_fwd_rot.restype = c_int
    lib.dlt_swa_fwd_rot.argtypes = fwd + [c_void_p, P64, c_void_p, P64, POINTER(SwaShape), POINTER(RopeDesc), c_void_p]
    lib.dlt_swa_bwd_rot.restype = c_int
    lib.dlt_swa_bwd_rot.argtypes = bwd + [POINTER(SwaShape), POINTER(RopeDesc), c_void_p]
    lib.dlt_swa_fwd_image.restype = c_int
    lib.dlt_swa_fwd_image.argtypes = fwd + [POINTER(SwaShape), POINTER(SwaTile), POINTER(RopeDesc), c_void_p]
    lib.dlt_swa_bwd_image.restype = c_int
    lib.dlt_swa_bwd_image.argtypes = bwd + [POINTER(SwaShape), POINTER(SwaTile), POINTER(RopeDesc), c_void_p]
    lib.dlt_swa_image_offsets.restype = c_int
    lib.dlt_swa_image_offsets.argtypes = [c_int32, c_int32, c_int32, c_int32, c_int64, c_int64, c_void_p, c_void_p]
    lib.dlt_flash_fwd.restype = c_int
    lib.dlt_flash_fwd.argtypes = fwd + [POINTER(FlashShape), c_void_p]
    lib.dlt_flash_bwd.restype = c_int
    lib.dlt_flash_bwd.argtypes = bwd + [POINTER(FlashShape), c_void_p]
    lib.dlt_debug_copy.restype = c_int
    lib.dlt_debug_copy.argtypes = [c_void_p, c_void_p, c_int64, c_void_p]
    lib.dlt_timing_enable.restype = c_int
    lib.dlt_timing_enable.argtypes = [c_int]
    lib.dlt_timing_collect.restype = c_int
    lib.dlt_timing_collect.argtypes = [POINTER(KernelTime), c_int, POINTER(c_int)]
    lib.dlt_dry_run.restype = c_int
    lib.dlt_dry_run.argtypes = [c_int]
    lib.dlt_last_kernel_family.restype = c_int
    lib.dlt_last_kernel_family.argtypes = []


def load():
    """Return the loaded library; raises if it has not been built."""
    global _lib
    if _lib is None:
        with _lock:
            if _lib is None:
                if not os.path.exists(LIB_PATH):
                    raise RuntimeError(
                        f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
                        f"or `make -C {CSRC_DIR}`. There is no CPU fallback.")
                lib = ctypes.CDLL(LIB_PATH)
                _declare(lib)
                _lib = lib
    return _lib


def check(rc: int) -> None:
    if rc != 0:
        raise DltError(rc, load().dlt_last_error().decode("utf-8", "replace"))


def timing_enable(on: bool) -> None:
    check(load().dlt_timing_enable(int(on)))


def timing_collect(max_records: int = 1 << 16):
    """[(kernel name, milliseconds)] for every launch since the last collect, in launch order."""
    buf = (KernelTime * max_records)()
    n = c_int(0)
    check(load().dlt_timing_collect(buf, max_records, ctypes.byref(n)))
    return [(KERNEL_NAMES[buf[i].kernel], float(buf[i].ms)) for i in range(min(n.value, max_records))]


def dtype_code(t: torch.Tensor) -> int:
    try:
        return _DTYPES[t.dtype]
    except KeyError:
        raise TypeError(f"unsupported dtype {t.dtype}; expected bfloat16, float16 or float32") from None


def strides(t: torch.Tensor):
    return (c_int64 * t.dim())(*t.stride())


def ptr(t: torch.Tensor) -> c_void_p:
    return c_void_p(t.data_ptr())


def stream_of(t: torch.Tensor) -> c_void_p:
    return c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def require_cuda(*tensors: torch.Tensor) -> None:
    dev = tensors[0].device
    for t in tensors:
        if not t.is_cuda:
            raise RuntimeError("dl_templates_amd runs on a ROCm GPU only: got a tensor on " + str(t.device))
        if t.device != dev:
            raise RuntimeError(f"all tensors must be on one device, got {dev} and {t.device}")


def rope_desc(idx: torch.Tensor, row_cs: torch.Tensor, col_cs: torch.Tensor, like: torch.Tensor = None,
              n_tokens: int = None):
    """(RopeDesc, keep-alive tuple).  Tables must be fp32 [len, R, 2] with a contiguous [R, 2] tail.

    ``like``: the tensor the rotation is applied to; idx and both tables must live on its device (the kernels
    dereference them: a host pointer would fault on the GPU instead of raising).  ``n_tokens``: idx must have
    exactly one entry per token."""
    if idx.dtype != torch.int32 or idx.dim() != 1 or not idx.is_contiguous():
        raise TypeError("idx must be a contiguous 1-D int32 tensor")
    if n_tokens is not None and idx.shape[0] != n_tokens:
        raise ValueError(f"idx has {idx.shape[0]} entries for {n_tokens} tokens")
    if like is not None:
        require_cuda(like, idx, row_cs, col_cs)
    tabs = []
    for t in (row_cs, col_cs):
        if t.dim() != 3 or t.shape[2] != 2:
            raise ValueError("cos/sin table must have shape [len, R, 2]")
        if t.dtype != torch.float32 or t.stride(2) != 1 or t.stride(1) != 2:
            t = t.float().contiguous()
        tabs.append(t)
    d = RopeDesc(idx.data_ptr(), tabs[0].data_ptr(), tabs[1].data_ptr(), tabs[0].stride(0), tabs[1].stride(0),
                 tabs[0].shape[1], tabs[0].shape[0], tabs[1].shape[0])
    return d, (idx, tabs[0], tabs[1])
