#!/usr/bin/env python3
"""Benchmark of the attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--quick]

One "step" is one forward + backward pass of the fused RoPE-2D + tiled 2D sliding-window
attention over one synthetic batch of benchmark config 3 (bf16, B=2, H=8, 64x64 token grid,
d=64, 13x13 window), inputs resident in HBM: the forward kernel rotates q and k as it loads its
tiles and keeps the rotated tensors, the backward kernels read those and rotate dq / dk back as they
store them (dlt_swa_fwd_rot / dlt_swa_bwd_rot).  `value` is the effective TFLOP/s of that
step (in-window FLOPs only: fwd 2*pairs*(dk+dv), bwd 2*pairs*(3dk+2dv)).  The JSON line also
carries the roofline of the dominant kernel (per-kernel HIP-event durations taken inside the
timed steps), the standalone RoPE-2D bandwidth (config 2), configs 4 / 5 as extras, and a CPU
baseline: the eager-PyTorch oracle of the same step timed on the host cores, whose outputs also check the GPU
results of the same seeded inputs (`accuracy`).  `ms_per_step` is the median of 5 repeats of >= 100 back-to-back
steps whatever --steps says (the mean over the requested steps is reported in `extra`).

Only one GPU is used; --gpus N with N > 1 exits with a message.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import math
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA, published
PEAK_HBM_GBPS = 8000.0     # MI355X HBM3E, published


def axis_count(t, w):
    w = min(w, t - 1)
    return t * (2 * w + 1) - w * (w + 1)


def swa_pairs(B, H, S, th, tw, wr, wc):
    return B * H * S * S * axis_count(th, wr) * axis_count(tw, wc)


def make_inputs(seed, B, H, Nq, Nk, dk, dv, dtype, device):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn((B, H, Nq, dk), generator=g)
    k = torch.randn((B, H, Nk, dk), generator=g)
    v = torch.randn((B, H, Nk, dv), generator=g)
    do = torch.randn((B, H, Nq, dv), generator=g)
    return [t.to(dtype).to(device) for t in (q, k, v, do)]


class Timer:
    """K back-to-back repetitions between two events on torch's current stream (the stream the
    library launches on)."""

    @staticmethod
    def run(fn, steps, warmup):
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        e0.record()
        for _ in range(steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        wall = (time.perf_counter() - t0) * 1e3 / steps
        return e0.elapsed_time(e1) / steps, wall


def median_of_repeats(fn, launches=100, repeats=5, warmup=10):
    """Median (and all samples) of `repeats` timings of `launches` back-to-back repetitions each."""
    samples = []
    for i in range(repeats):
        ms, _ = Timer.run(fn, launches, warmup if i == 0 else 0)
        samples.append(ms)
    srt = sorted(samples)
    return srt[len(srt) // 2], samples


def kernel_breakdown(fn, steps):
    """Average per-kernel duration (ms) over `steps` eager repetitions, from HIP events recorded
    around every launch on the launch stream."""
    from dl_templates_amd import _lib
    torch.cuda.synchronize()
    _lib.timing_enable(True)
    try:
        for _ in range(steps):
            fn()
        torch.cuda.synchronize()
        rec = _lib.timing_collect()
    finally:
        _lib.timing_enable(False)
    acc = {}
    for name, ms in rec:
        s = acc.setdefault(name, [0.0, 0])
        s[0] += ms
        s[1] += 1
    return {k: {"avg_ms": v[0] / v[1], "launches_per_step": v[1] / steps} for k, v in acc.items()}


def try_graph(wl, steps, warmup):
    """Replay `len(wl.calls)` steps (one per input set) from a captured HIP graph, so that host
    launch cost is out of the picture; returns (ms per step over the requested steps, ms per step as the median of 5
    repeats of >= 100 steps: the protocol of the eager headline) or (None, None) if capture fails.  The
    library launches on the stream it is handed, so the capture stream is passed explicitly."""
    try:
        s = torch.cuda.Stream()
        s.wait_stream(torch.cuda.current_stream())
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        nsets = len(wl.calls)
        with torch.cuda.graph(g, stream=s):
            wl.stream.value = torch.cuda.current_stream().cuda_stream
            for _ in range(nsets):
                wl.step()
        wl.stream.value = torch.cuda.current_stream().cuda_stream
        reps = max(steps // nsets, 1)
        ms, _ = Timer.run(g.replay, reps, max(warmup // nsets, 1))
        med, _ = median_of_repeats(g.replay, launches=max(100, steps) // nsets, repeats=5, warmup=2)
        return ms / nsets, med / nsets
    except Exception as exc:  # pragma: no cover - depends on the runtime
        wl.stream.value = torch.cuda.current_stream().cuda_stream
        print(f"[bench] graph capture unavailable: {exc}", file=sys.stderr)
        return None, None


# ------------------------------------------------------------------------------------------ SWA
class SwaWorkload:
    def __init__(self, name, B, H, th, tw, W, d, fused_rope, nsets, seed=0, dtype=torch.bfloat16, b_size=1, scale=None,
                 keep_rotated=True):
        from dl_templates_amd import _lib, tiled_swa
        from dl_templates_amd.rope2d import FusedRotaryPositionEncodingContext as Ctx
        from dl_templates_amd.fused_rope2d import FusedInplaceRotaryPositionEncoding2D as Rope
        self.name, self.B, self.H, self.th, self.tw, self.W, self.d = name, B, H, th, tw, W, d
        # fused rotation: the forward pass keeps the rotated q, k for the backward pass (dlt_swa_fwd_rot /
        # dlt_swa_bwd_rot, what TiledSwaRope does by default) or every tile load of the backward kernels
        # rotates again (dlt_swa_fwd / dlt_swa_bwd with the rotary operands)
        self.keep_rotated = bool(fused_rope and keep_rotated)
        dev = torch.device("cuda:0")
        N = th * tw * b_size
        self.sets = []
        for i in range(nsets):
            q, k, v, do = make_inputs(seed + i, B, H, N, N, d, d, dtype, dev)
            o = torch.empty_like(v)
            lse = torch.empty((B, H, N), dtype=torch.float32, device=dev)
            delta = torch.empty_like(lse)
            dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
            rot = (torch.empty_like(q), torch.empty_like(k)) if self.keep_rotated else (None, None)
            self.sets.append((q, k, v, do, o, lse, delta, dq, dk, dv) + rot)
        self.shape = _lib.SwaShape(B, H, b_size, th, tw, W, W, d, d, scale if scale is not None else 1.0 / math.sqrt(d),
                                   _lib.dtype_code(self.sets[0][0]))
        self.rope = None
        if fused_rope:
            g = torch.Generator().manual_seed(seed + 1000)
            idx = Rope.encode_idx(th, tw).clone()
            idx[torch.rand(N, generator=g) < 0.05] = -1
            self.idx = idx.to(dev)
            self.rcs = Ctx(16, th).cs_components.to(dev)
            self.ccs = Ctx(16, tw).cs_components.to(dev)
            self.rope, self._keep = _lib.rope_desc(self.idx, self.rcs, self.ccs)
        self.lib = _lib.load()
        self._lib = _lib
        self.stream = _lib.stream_of(self.sets[0][0])
        self._fwd = self.lib.dlt_swa_fwd_rot if self.keep_rotated else self.lib.dlt_swa_fwd
        self._bwd = self.lib.dlt_swa_bwd_rot if self.keep_rotated else self.lib.dlt_swa_bwd
        self.calls = [self._build_calls(s) for s in self.sets]
        self.i = 0
        self.pairs = swa_pairs(B, H, b_size, th, tw, W, W)
        self.flops_fwd = 2 * self.pairs * (d + d)
        self.flops_bwd = 2 * self.pairs * (3 * d + 2 * d)

    def _build_calls(self, s):
        L = self._lib
        q, k, v, do, o, lse, delta, dq, dk, dv, q_rot, k_rot = s
        fwd = (L.ptr(q), L.strides(q), L.ptr(k), L.strides(k), L.ptr(v), L.strides(v), L.ptr(o), L.strides(o),
               L.ptr(lse), L.strides(lse))
        if self.keep_rotated:
            fwd += (L.ptr(q_rot), L.strides(q_rot), L.ptr(k_rot), L.strides(k_rot))
        fwd += (self.shape, self.rope, self.stream)
        qb, kb = (q_rot, k_rot) if self.keep_rotated else (q, k)
        bwd = (L.ptr(qb), L.strides(qb), L.ptr(kb), L.strides(kb), L.ptr(v), L.strides(v), L.ptr(o), L.strides(o),
               L.ptr(do), L.strides(do), L.ptr(lse), L.ptr(delta), L.strides(lse), L.ptr(dq), L.strides(dq),
               L.ptr(dk), L.strides(dk), L.ptr(dv), L.strides(dv), self.shape, self.rope, self.stream)
        return fwd, bwd

    def step(self):
        fwd, bwd = self.calls[self.i % len(self.calls)]
        self.i += 1
        rc = self._fwd(*fwd)
        rc = rc or self._bwd(*bwd)
        if rc:
            self._lib.check(rc)

    def fwd_only(self):
        fwd, _ = self.calls[self.i % len(self.calls)]
        self.i += 1
        rc = self._fwd(*fwd)
        if rc:
            self._lib.check(rc)

    def kernel_flops(self):
        d = self.d
        return {"attn_fwd": self.flops_fwd, "attn_bwd_kv": 2 * self.pairs * (2 * d + 2 * d), "attn_bwd_q": 2 * self.pairs * d}


class FlashWorkload:
    def __init__(self, B, H, Lq, Lk, dk, dv, seed=0, dtype=torch.bfloat16, causal=False, scale=None):
        from dl_templates_amd import _lib
        dev = torch.device("cuda:0")
        q, k, v, do = make_inputs(seed, B, H, Lq, Lk, dk, dv, dtype, dev)
        o = torch.empty((B, H, Lq, dv), dtype=dtype, device=dev)
        lse = torch.empty((B, H, Lq), dtype=torch.float32, device=dev)
        delta = torch.empty_like(lse)
        dq, dkk, dvv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        self.keep = (q, k, v, do, o, lse, delta, dq, dkk, dvv)
        L = _lib
        shape = L.FlashShape(B, H, Lq, Lk, dk, dv, scale if scale is not None else 1.0 / math.sqrt(dk), int(causal), L.dtype_code(q))
        st = L.stream_of(q)
        self.fwd = (L.ptr(q), L.strides(q), L.ptr(k), L.strides(k), L.ptr(v), L.strides(v), L.ptr(o), L.strides(o),
                    L.ptr(lse), L.strides(lse), shape, st)
        self.bwd = (L.ptr(q), L.strides(q), L.ptr(k), L.strides(k), L.ptr(v), L.strides(v), L.ptr(o), L.strides(o),
                    L.ptr(do), L.strides(do), L.ptr(lse), L.ptr(delta), L.strides(lse), L.ptr(dq), L.strides(dq),
                    L.ptr(dkk), L.strides(dkk), L.ptr(dvv), L.strides(dvv), shape, st)
        self.lib, self._lib = L.load(), L
        pairs = B * H * Lq * Lk * (0.5 if causal else 1.0)  # the reference's convention for causal (src/flash_attn.py:608-614)
        self.flops_fwd = 2 * pairs * (dk + dv)
        self.flops_bwd = 2 * pairs * (3 * dk + 2 * dv)

    def step(self):
        rc = self.lib.dlt_flash_fwd(*self.fwd) or self.lib.dlt_flash_bwd(*self.bwd)
        if rc:
            self._lib.check(rc)

    def fwd_only(self):
        rc = self.lib.dlt_flash_fwd(*self.fwd)
        if rc:
            self._lib.check(rc)


# ------------------------------------------------------------------------------------------ RoPE
def bench_rope(steps, warmup, R=8):
    """Config 2 (R = 8): B=4, H=8, 64x64, d=64, first 32 dims rotated, 5% no-PE, q and k in one launch.
    `cold` cycles through > 512 MB of distinct (q, k) pairs so that the 256 MB infinity cache
    cannot hold the working set; `hot` reuses one pair.  R = 16 is the same launch with the whole 64-dim row rotated:
    every byte of a fetched 128-byte line is used, so algorithmic and real traffic coincide."""
    from dl_templates_amd import _lib
    from dl_templates_amd.rope2d import FusedRotaryPositionEncodingContext as Ctx
    from dl_templates_amd.fused_rope2d import FusedInplaceRotaryPositionEncoding2D as Rope
    dev = torch.device("cuda:0")
    B, H, N, C = 4, 8, 4096, 64
    g = torch.Generator().manual_seed(2)
    idx = Rope.encode_idx(64, 64).clone()
    idx[torch.rand(N, generator=g) < 0.05] = -1
    n_pe = int((idx >= 0).sum())
    idx = idx.to(dev)
    rcs, ccs = Ctx(2 * R, 64).cs_components.to(dev), Ctx(2 * R, 64).cs_components.to(dev)
    desc, keep = _lib.rope_desc(idx, rcs, ccs)
    lib = _lib.load()
    nbuf = 17  # 17 * 2 * 16.8 MB = 570 MB
    bufs = [(torch.randn(B * H, N, C, generator=g).to(torch.bfloat16).to(dev),
             torch.randn(B * H, N, C, generator=g).to(torch.bfloat16).to(dev)) for _ in range(nbuf)]
    st = _lib.stream_of(idx)
    calls = [(_lib.ptr(q), _lib.strides(q), B * H, _lib.ptr(k), _lib.strides(k), B * H, N, C, desc, 0, _lib.DLT_BF16, st)
             for q, k in bufs]
    state = {"i": 0}

    def cold():
        rc = lib.dlt_rope2d_pair(*calls[state["i"] % nbuf])
        state["i"] += 1
        if rc:
            _lib.check(rc)

    def hot():
        rc = lib.dlt_rope2d_pair(*calls[0])
        if rc:
            _lib.check(rc)

    # algorithmic bytes: read + write of the 4R rotated dims of tokens with a rotated axis, idx once, x2 tensors
    alg_bytes = 2 * (2 * 2 * (B * H) * n_pe * 4 * R) + 4 * N
    # real traffic: reads fetch whole 128-byte lines, writes carry the bytes stored.  With R = 8 only the first 64 bytes of
    # each 128-byte token row rotate, so a rotated token costs 128 bytes read + 64 written = 1.5 x its algorithmic bytes
    # (the counters in profiles/ read 1.56 x for the launch, tables and idx included); with 4 R = C the two coincide
    real_bytes = 2 * (2 * (B * H) * n_pe * (max(C, 4 * R) + 4 * R)) + 4 * N
    line_factor = real_bytes / alg_bytes
    out = {"alg_bytes": alg_bytes, "n_pe_tokens": n_pe, "rotary_pairs_per_axis": R,
           "real_bytes_over_alg_bytes": line_factor}
    for name, fn in (("cold", cold), ("hot", hot)):
        ms_ev, _ = Timer.run(fn, steps * 5, warmup * 5)
        kb = kernel_breakdown(fn, steps * 5)
        kms = kb["rope2d"]["avg_ms"]
        out[name] = {"us_per_launch_back_to_back": ms_ev * 1e3, "us_kernel_events": kms * 1e3,
                     "gbps": alg_bytes / (kms * 1e-3) / 1e9, "frac_of_hbm_peak": alg_bytes / (kms * 1e-3) / 1e9 / PEAK_HBM_GBPS,
                     "gbps_back_to_back": alg_bytes / (ms_ev * 1e-3) / 1e9,
                     "real_traffic_gbps_back_to_back": alg_bytes * line_factor / (ms_ev * 1e-3) / 1e9}
    del keep
    return out


# ------------------------------------------------------------------------------------------ CPU baseline
def gpu_results_for_accuracy():
    """GPU outputs the CPU-baseline leg checks: the fused config-3 step on the inputs of seed 0 (the same draws
    make_qkv(0, ...) yields on the host), config-2 rotation of a seeded tensor, neighbour sets and no-PE masks."""
    from dl_templates_amd import fused_rope2d, tiled_swa
    from dl_templates_amd.rope2d import FusedRotaryPositionEncodingContext as Ctx
    from dl_templates_amd.fused_rope2d import FusedInplaceRotaryPositionEncoding2D as Rope
    dev = torch.device("cuda:0")
    B, H, th, tw, W, d = 2, 8, 64, 64, 6, 64
    N = th * tw
    q, k, v, do = make_inputs(0, B, H, N, N, d, d, torch.bfloat16, dev)
    g = torch.Generator().manual_seed(1000)
    idx = Rope.encode_idx(th, tw).clone()
    idx[torch.rand(N, generator=g) < 0.05] = -1
    rcs, ccs = Ctx(16, th).cs_components.to(dev), Ctx(16, tw).cs_components.to(dev)
    qg, kg, vg = (t.detach().requires_grad_(True) for t in (q, k, v))
    o = tiled_swa.TiledSwaRope.apply(qg, kg, vg, idx.to(dev), rcs, ccs, 1, th, tw, W, W, 1.0 / math.sqrt(d))
    o.backward(do)
    out = {"idx": idx, "o": o.detach().float().cpu(), "dq": qg.grad.float().cpu(), "dk": kg.grad.float().cpu(),
           "dv": vg.grad.float().cpu()}
    # config 2: B=4, H=8 -> 32 batch rows, 64 x 64 tokens, C = 64, R = 8, 5 % no-PE
    g2 = torch.Generator().manual_seed(2)
    idx2 = Rope.encode_idx(64, 64).clone()
    idx2[torch.rand(N, generator=g2) < 0.05] = -1
    x = torch.randn(32, N, 64, generator=g2).to(torch.bfloat16)
    xr = fused_rope2d.RotaryPE2D.apply(x.to(dev).clone(), idx2.to(dev), rcs, ccs)
    out.update({"idx2": idx2, "x": x, "x_rot": xr.cpu(), "rcs": rcs.cpu(), "ccs": ccs.cpu()})
    out["neighbors"] = tiled_swa.swa_neighbors(16, 16, 3, 3).cpu().numpy()
    from dl_templates_amd import _lib
    bits = torch.empty(N, dtype=torch.uint8, device=dev)
    _lib.check(_lib.load().dlt_rope_pe_mask(_lib.ptr(idx2.to(dev)), N, _lib.ptr(bits), _lib.stream_of(bits)))
    out["pe_bits"] = bits.cpu().numpy()
    return out


def cpu_baseline_c3(gpu):
    """The CPU leg: the oracle (eager PyTorch, fp32) of the same fused config-3 step on the host cores, three
    repetitions after a warm-up on a quarter of the heads; its outputs then serve as the checker for the GPU
    results of the same seeded inputs (`gpu`, from gpu_results_for_accuracy): returns (cpu_baseline, accuracy)."""
    import numpy as np
    from oracle import attn_oracle as orc
    B, H, th, tw, W, d = 2, 8, 64, 64, 6, 64
    N = th * tw
    q, k, v, do = orc.make_qkv(0, B, H, N, N, d, d, torch.bfloat16)
    q, k, v, do = (t.float() for t in (q, k, v, do))
    idx = gpu["idx"]
    rcs, ccs = orc.rope_tables(8, th), orc.rope_tables(8, tw)
    args = (idx, rcs, ccs, 1, th, tw, W, W, 1.0 / math.sqrt(d))
    orc.rope_swa_grads(q[:, :2], k[:, :2], v[:, :2], do[:, :2], *args)
    times = []
    for _ in range(3):
        t0 = time.perf_counter()
        o_w, dq_w, dk_w, dv_w = orc.rope_swa_grads(q, k, v, do, *args)
        times.append(time.perf_counter() - t0)
    dt = sorted(times)[1]
    pairs = swa_pairs(B, H, 1, th, tw, W, W)
    flops = 2 * pairs * (d + d) + 2 * pairs * (5 * d)
    cpu = {"value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
           "sample": f"whole config-3 step (B=2,H=8,64x64,d=64,13x13, fp32 eager masked SDPA + autograd), median of 3 repetitions "
                     f"({', '.join(f'{t * 1e3:.0f}' for t in times)} ms)",
           "ms_per_step": dt * 1e3, "host_cpus": os.cpu_count()}

    def rel(got, want):
        return ((got - want).abs().max() / want.abs().max()).item()

    def frob(got, want):
        return ((got - want).norm() / want.norm()).item()

    y = orc.rope2d_ref(gpu["x"].float(), gpu["idx2"], gpu["rcs"], gpu["ccs"]).to(torch.bfloat16)
    acc = {
        "workload": "config 3 fused step on the inputs of seed 0 (B=2, H=8: all of it), config 2 rotation, 16x16 grid 7x7 window "
                    "neighbour sets, config 2 no-PE mask; checked against the CPU oracle outside the timed region",
        "fwd_max_abs": (gpu["o"] - o_w).abs().max().item(), "fwd_max_abs_bar": 2e-2,
        "dq_rel": rel(gpu["dq"], dq_w), "dk_rel": rel(gpu["dk"], dk_w), "dv_rel": rel(gpu["dv"], dv_w), "grad_rel_bar": 5e-2,
        "dq_frobenius_rel": frob(gpu["dq"], dq_w), "dk_frobenius_rel": frob(gpu["dk"], dk_w), "dv_frobenius_rel": frob(gpu["dv"], dv_w),
        "rope_max_bf16_ulp": int(orc.bf16_ulp_diff(gpu["x_rot"], y).max()), "rope_ulp_bar": 1,
        "neighbor_sets_bit_exact": bool(np.array_equal(gpu["neighbors"], orc.neighbor_mask(16, 16, 3, 3))),
        "no_pe_mask_bit_exact": bool(np.array_equal(gpu["pe_bits"], orc.pe_mask(gpu["idx2"].numpy()))),
    }
    acc["within_bars"] = bool(acc["fwd_max_abs"] <= 2e-2 and max(acc["dq_rel"], acc["dk_rel"], acc["dv_rel"]) <= 5e-2 and
                              acc["rope_max_bf16_ulp"] <= 1 and acc["neighbor_sets_bit_exact"] and acc["no_pe_mask_bit_exact"])
    return cpu, acc


def calibration_copy():
    """A 64 MiB device copy through the library's plain copy kernel: a launch of exactly known
    traffic, present in every profiler run of this script so that FETCH_SIZE / WRITE_SIZE
    readings of the other kernels can be scaled by what the counters report for it."""
    from dl_templates_amd import _lib
    a = torch.empty(64 << 20, dtype=torch.uint8, device="cuda:0")
    b = torch.empty_like(a)
    for _ in range(2):
        _lib.check(_lib.load().dlt_debug_copy(_lib.ptr(b), _lib.ptr(a), a.numel(), _lib.stream_of(a)))
    torch.cuda.synchronize()


def copy_bandwidth():
    """What the memory system sustains for a plain copy (read + write bytes per second): 64 MiB
    (resident in the 256 MB infinity cache after the first pass), 1 GiB (HBM), and 24 MiB copies from
    cold buffers (a launch of the size of the RoPE benchmark)."""
    from dl_templates_amd import _lib
    lib = _lib.load()
    out = {}
    for name, nbytes, reps in (("64MiB_cache_resident", 64 << 20, 20), ("1GiB_hbm", 1 << 30, 5)):
        a = torch.empty(nbytes, dtype=torch.uint8, device="cuda:0")
        b = torch.empty_like(a)
        st = _lib.stream_of(a)
        fn = lambda: _lib.check(lib.dlt_debug_copy(_lib.ptr(b), _lib.ptr(a), nbytes, st))
        ms, _ = Timer.run(fn, reps, 2)
        ms_t, _ = Timer.run(lambda: b.copy_(a), reps, 2)   # PyTorch's own device copy: an independent yardstick
        out[name] = {"ms": ms, "gbps_read_plus_write": 2 * nbytes / (ms * 1e-3) / 1e9,
                     "torch_copy_ms": ms_t, "torch_copy_gbps_read_plus_write": 2 * nbytes / (ms_t * 1e-3) / 1e9}
        del a, b
    # a copy with the real traffic of one RoPE C2 launch (about 48 MiB), cold: 13 buffer pairs cycled (624 MiB)
    nbytes, npairs = 24 << 20, 13
    bufs = [(torch.empty(nbytes, dtype=torch.uint8, device="cuda:0"), torch.empty(nbytes, dtype=torch.uint8, device="cuda:0"))
            for _ in range(npairs)]
    st = _lib.stream_of(bufs[0][0])
    state = {"i": 0}

    def cold():
        a, b = bufs[state["i"] % npairs]
        state["i"] += 1
        _lib.check(lib.dlt_debug_copy(_lib.ptr(b), _lib.ptr(a), nbytes, st))

    ms, _ = Timer.run(cold, 5 * npairs, npairs)

    def cold_torch():
        a, b = bufs[state["i"] % npairs]
        state["i"] += 1
        b.copy_(a)

    ms_t, _ = Timer.run(cold_torch, 5 * npairs, npairs)
    out["24MiB_cold"] = {"ms": ms, "gbps_read_plus_write": 2 * nbytes / (ms * 1e-3) / 1e9,
                         "torch_copy_ms": ms_t, "torch_copy_gbps_read_plus_write": 2 * nbytes / (ms_t * 1e-3) / 1e9}
    return out


def recorded_traffic(kernel):
    """HBM bytes per launch of `kernel` on the C3 workload as recorded under profiles/ (two
    rocprofv3 --pmc runs of this script, scaled by the calibration copy); None if absent."""
    path = os.path.join(ROOT, "profiles", "c3_kernels_hbm_traffic.json")
    try:
        with open(path) as f:
            return json.load(f).get(kernel, {}).get("hbm_bytes_per_launch")
    except (OSError, ValueError):
        return None


def image_layout_demo(steps):
    from dl_templates_amd import tiled_swa
    B, H, th, tw, bh, bw, d = 4, 8, 64, 64, 4, 4, 32   # the demo's tiles and head dim on a 256 x 256 image
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(3)
    img = [torch.randn((B, th * bh, tw * bw, H, d), generator=g).to(torch.float16).to(dev) for _ in range(4)]
    qi, ki, vi, doi = img

    def to_tokens(x):   # [B, IH, IW, H, D] -> [B, H, N, D], a real copy
        return x.reshape(B, th, bh, tw, bw, H, d).permute(0, 5, 1, 3, 2, 4, 6).reshape(B, H, th * tw * bh * bw, d)

    def to_image(x):
        return x.reshape(B, H, th, tw, bh, bw, d).permute(0, 2, 4, 3, 5, 1, 6).reshape(B, th * bh, tw * bw, H, d)

    def direct():
        q, k, v = (t.detach().requires_grad_(True) for t in (qi, ki, vi))
        tiled_swa.TiledSwaImage.apply(q, k, v, bh, bw, 1, 1, 0.25).backward(doi)
        return q.grad, k.grad, v.grad

    def converted():
        q, k, v = (to_tokens(t).requires_grad_(True) for t in (qi, ki, vi))
        o = tiled_swa.TiledSwa.apply(q, k, v, bh * bw, th, tw, 1, 1, 0.25)
        o.backward(to_tokens(doi))
        return to_image(o), to_image(q.grad), to_image(k.grad), to_image(v.grad)

    ms_direct, _ = Timer.run(direct, steps, 3)
    ms_conv, _ = Timer.run(converted, steps, 3)
    return {"ms_image_entry_points": ms_direct, "ms_convert_run_convert_back": ms_conv,
            "workload": "B=4 H=8, 256x256 pixel image, 4x4-pixel tiles, d=32, 3x3 tile window, fp16, fwd+bwd"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--quick", action="store_true", help="skip the extra configs and the CPU baseline")
    ap.add_argument("--workload", choices=("all", "c4", "c4b", "c5"), default="all",
                    help="c4 / c4b / c5: run only config 4 (128x128 / 96x160) or config 5 and print its timing (for profiler runs)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the hot path shards over batch*heads with no exchange); "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(2)
    torch.cuda.set_device(0)
    K, W = args.steps, args.warmup
    calibration_copy()
    if args.workload != "all":
        # one extra config alone, for rocprofv3 runs: the calibration copy above, then W + K steps
        if args.workload == "c5":
            w = FlashWorkload(2, 16, 4096, 8192, 64, 128)
        else:
            th, tw = (128, 128) if args.workload == "c4" else (96, 160)
            w = SwaWorkload(args.workload, 1, 16, th, tw, 10, 128, fused_rope=False, nsets=1)
        ms, _ = Timer.run(w.step, K, W)
        kbw = kernel_breakdown(w.step, max(K // 2, 2))
        fl = w.flops_fwd + w.flops_bwd
        print(json.dumps({"workload": args.workload, "ms_per_step": ms, "eff_tflops": fl / (ms * 1e-3) / 1e12,
                          "frac_mfma_peak": fl / (ms * 1e-3) / 1e12 / PEAK_BF16_TFLOPS,
                          "kernels_ms": {k_: v_["avg_ms"] for k_, v_ in kbw.items()}}))
        return

    # ---- main workload: config 3, fused RoPE, 4 input sets cycled (about 400 MB touched per cycle)
    wl = SwaWorkload("C3", 2, 8, 64, 64, 6, 64, fused_rope=True, nsets=4)
    ms_eager, wall_eager = Timer.run(wl.step, K, W)
    kb = kernel_breakdown(wl.step, max(K, 20))
    ms_graph, ms_graph_median = try_graph(wl, K, W)
    # headline: median of 5 repeats of >= 100 back-to-back steps (eager launches), whatever --steps says; the mean over the
    # K requested steps and the HIP-graph replay of the same steps are reported beside it
    ms_median, ms_samples = median_of_repeats(wl.step, launches=max(100, K), repeats=5, warmup=W)
    ms_step = ms_median
    flops_step = wl.flops_fwd + wl.flops_bwd
    value = flops_step / (ms_step * 1e-3) / 1e12

    kflops = wl.kernel_flops()
    # the dominant kernel: the longest one; kernels within 3 % of it (run-to-run noise) count as equally long, and among
    # those the one that does the most algorithmic work stands for the step
    longest = max(kb[k]["avg_ms"] for k in kb if k in kflops)
    dom = max((k for k in kb if k in kflops and kb[k]["avg_ms"] >= 0.97 * longest), key=lambda k: kflops[k])
    # A pair of HIP events around a launch adds the markers' own cost to every kernel: the kernels of a step, bracketed,
    # sum to more than the step takes back to back without markers.  That excess, spread evenly over the step's launches,
    # is taken off again, so that `avg_launch_ms` is the kernel's share of the un-instrumented step (what rocprofv3's
    # kernel trace in profiles/ shows as its average duration); the raw bracketed figure stays beside it.
    n_launch = sum(v["launches_per_step"] for k, v in kb.items() if k in kflops)
    bracketed_sum = sum(v["avg_ms"] * v["launches_per_step"] for k, v in kb.items() if k in kflops)
    marker_ms = max(0.0, (bracketed_sum - ms_step) / n_launch)
    dom_ms = kb[dom]["avg_ms"] - marker_ms
    ach = kflops[dom] / (dom_ms * 1e-3) / 1e12
    roofline = {"bound": "mfma", "kernel": dom, "achieved": ach, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                "frac": ach / PEAK_BF16_TFLOPS, "traffic": recorded_traffic(dom),
                "traffic_source": "recorded in profiles/c3_kernels_hbm_traffic.json (rocprofv3 --pmc runs of this script), not measured by this run",
                "avg_launch_ms": dom_ms, "avg_launch_ms_event_bracketed": kb[dom]["avg_ms"], "event_marker_ms_per_launch": marker_ms,
                "alg_flops_per_launch": kflops[dom],
                "step": {"achieved": value, "frac": value / PEAK_BF16_TFLOPS, "ms": ms_step, "alg_flops": flops_step}}
    kernels = {}
    for k_, v_ in kb.items():
        kernels[k_] = {"avg_ms": v_["avg_ms"]}
        if k_ in kflops:
            kernels[k_]["eff_tflops"] = kflops[k_] / (v_["avg_ms"] * 1e-3) / 1e12
            kernels[k_]["frac_mfma_peak"] = kernels[k_]["eff_tflops"] / PEAK_BF16_TFLOPS

    extra = {"ms_per_step_mean_of_requested_steps": ms_eager, "ms_per_step_eager_wall": wall_eager, "ms_per_step_graph": ms_graph,
             "ms_per_step_graph_median_of_5x100": ms_graph_median,
             "ms_per_step_median_of_5x100": ms_median, "ms_per_step_samples_5x100": ms_samples,
             "step_source": "median of 5 repeats of >= 100 eager back-to-back steps",
             "frac_mfma_peak_effective": value / PEAK_BF16_TFLOPS, "kernels": kernels,
             "hbm_floor_ms": 101e6 / (PEAK_HBM_GBPS * 1e9) * 1e3}

    rope = bench_rope(K, W)
    extra["rope2d_c2"] = rope
    extra["rope2d_whole_row_r16"] = bench_rope(K, W, R=16)
    extra["copy_bandwidth"] = copy_bandwidth()
    # the rotation against what a plain copy sustains on this box: real traffic of a cold launch over the 1 GiB copy rate
    # (HBM, far beyond the caches) and over a cold copy of the launch's own size
    cb = extra["copy_bandwidth"]
    for key in ("rope2d_c2", "rope2d_whole_row_r16"):
        r_ = extra[key]["cold"]
        r_["frac_of_1GiB_copy_rate"] = r_["real_traffic_gbps_back_to_back"] / cb["1GiB_hbm"]["gbps_read_plus_write"]
        r_["frac_of_cold_copy_of_same_size"] = r_["real_traffic_gbps_back_to_back"] / cb["24MiB_cold"]["gbps_read_plus_write"]

    # the extra configs: long enough runs (tens of milliseconds of GPU time behind a warm-up) that the clock ramp after an
    # idle phase does not weigh on the mean
    XK, XW = max(K, 40), 8
    if not args.quick:
        # the same step when nothing but the caller's q, k is kept: every K / Q tile load of the backward
        # kernels rotates again (dlt_swa_fwd / dlt_swa_bwd with the rotary operands)
        wl2 = SwaWorkload("C3", 2, 8, 64, 64, 6, 64, fused_rope=True, nsets=4, keep_rotated=False)
        ms2, _ = Timer.run(wl2.step, K, W)
        kb2 = kernel_breakdown(wl2.step, K)
        extra["C3_rotation_in_every_tile_load"] = {"ms_per_step_eager_events": ms2, "eff_tflops": flops_step / (ms2 * 1e-3) / 1e12,
                                                   "kernels_ms": {k_: v_["avg_ms"] for k_, v_ in kb2.items()}}
        del wl2
        for name, (B, H, th, tw, Wn, d) in {"C4_128x128": (1, 16, 128, 128, 10, 128), "C4_96x160": (1, 16, 96, 160, 10, 128)}.items():
            w4 = SwaWorkload(name, B, H, th, tw, Wn, d, fused_rope=False, nsets=1)
            ms4, _ = Timer.run(w4.step, XK, XW)
            kb4 = kernel_breakdown(w4.step, 10)
            f4 = w4.flops_fwd + w4.flops_bwd
            extra[name] = {"ms_per_step": ms4, "eff_tflops": f4 / (ms4 * 1e-3) / 1e12,
                           "frac_mfma_peak": f4 / (ms4 * 1e-3) / 1e12 / PEAK_BF16_TFLOPS,
                           "kernels_ms": {k_: v_["avg_ms"] for k_, v_ in kb4.items()}}
            del w4
        # the reference's own demo shape (src/tiled_swa.py:736-750): 16-token tiles, generic kernels
        wd = SwaWorkload("ref_demo", 4, 8, 16, 16, 1, 32, fused_rope=False, nsets=1, dtype=torch.float16, b_size=16, scale=0.25)
        msd, _ = Timer.run(wd.step, XK, XW)
        fd = wd.flops_fwd + wd.flops_bwd
        extra["ref_demo_b16"] = {"ms_per_step": msd, "eff_tflops": fd / (msd * 1e-3) / 1e12,
                                 "workload": "B=4 H=8 16x16 tiles of 16 tokens, d=32, 3x3 window, fp16, fwd+bwd (src/tiled_swa.py:736-750)"}
        del wd
        # the demo's tiles with q, k, v, dO kept as images [B, IH, IW, heads, D] (4 x 4 pixel tiles):
        # the image entry points against converting to the token layout and back around the operator
        # (src/tiled_swa.py:753-755), both through the autograd functions of the package
        extra["ref_demo_image_layout"] = image_layout_demo(max(K // 5, 3))
        # larger tiles: B=2, H=8, 16x16 tiles of 64 tokens (N = 16384), d=64, 3x3 tile window, bf16
        wt = SwaWorkload("tiles_b64", 2, 8, 16, 16, 1, 64, fused_rope=False, nsets=1, b_size=64)
        mst, _ = Timer.run(wt.step, XK, XW)
        kbt = kernel_breakdown(wt.step, 10)
        ft = wt.flops_fwd + wt.flops_bwd
        extra["tiles_b64_d64"] = {"ms_per_step": mst, "eff_tflops": ft / (mst * 1e-3) / 1e12,
                                  "frac_mfma_peak": ft / (mst * 1e-3) / 1e12 / PEAK_BF16_TFLOPS,
                                  "kernels_ms": {k_: v_["avg_ms"] for k_, v_ in kbt.items()},
                                  "workload": "B=2 H=8 16x16 tiles of 64 tokens, d=64, 3x3 tile window, bf16, fwd+bwd"}
        del wt
        # the shape the reference publishes flash numbers for (B=4, H=32, d=64, fp16, sm_scale 1.3,
        # src/flash_attn.py:548,580-586; its CSVs name no hardware), at N_CTX = 4096
        ref = {}
        for causal in (False, True):
            wr = FlashWorkload(4, 32, 4096, 4096, 64, 64, dtype=torch.float16, causal=causal, scale=1.3)
            ms_f, _ = Timer.run(wr.fwd_only, XK, XW)
            ms_s, _ = Timer.run(wr.step, XK, XW)
            ref["causal" if causal else "non_causal"] = {
                "fwd_ms": ms_f, "fwd_tflops": wr.flops_fwd / (ms_f * 1e-3) / 1e12,
                "bwd_ms": ms_s - ms_f, "bwd_tflops": wr.flops_bwd / ((ms_s - ms_f) * 1e-3) / 1e12}
            del wr
        ref["published_triton_fp16_unstated_hw_tflops"] = {"fwd_non_causal": 73.56, "fwd_causal": 71.11, "bwd_causal": 38.22}
        extra["flash_ref_b4_h32_d64_n4096_fp16"] = ref
        w5 = FlashWorkload(2, 16, 4096, 8192, 64, 128)
        ms5, _ = Timer.run(w5.step, XK, XW)
        kb5 = kernel_breakdown(w5.step, 10)
        f5 = w5.flops_fwd + w5.flops_bwd
        extra["C5_flash"] = {"ms_per_step": ms5, "eff_tflops": f5 / (ms5 * 1e-3) / 1e12,
                             "frac_mfma_peak": f5 / (ms5 * 1e-3) / 1e12 / PEAK_BF16_TFLOPS,
                             "kernels_ms": {k_: v_["avg_ms"] for k_, v_ in kb5.items()}}
        del w5

    cpu, accuracy = (None, None) if args.quick else cpu_baseline_c3(gpu_results_for_accuracy())

    line = {
        "metric": "swa2d_fwd_bwd_effective_tflops", "value": value, "unit": "TFLOP/s", "n_gpus": 1, "steps": K,
        "warmup": W, "ms_per_step": ms_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "C3: fused RoPE-2D + tiled 2D SWA fwd+bwd, B=2 H=8 64x64 grid b_size=1 d=64 13x13 window, "
                               "bf16, 5% no-PE tokens, 4 input sets cycled; rotated q, k kept by the forward pass for the backward pass",
                   "peak_bf16_tflops": PEAK_BF16_TFLOPS, "peak_hbm_gbps": PEAK_HBM_GBPS},
        "roofline": roofline, "cpu_baseline": cpu, "accuracy": accuracy,
        "rope2d_gbps": rope["cold"]["gbps"], "rope2d_frac_hbm": rope["cold"]["frac_of_hbm_peak"],
        "extra": extra,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
