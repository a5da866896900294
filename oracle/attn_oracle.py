"""CPU oracle for the attention hot path (TEST INFRASTRUCTURE - NOT PRODUCT CODE).

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this module.  The product path (``dl_templates_amd``)
never imports it and never falls back to it: when the HIP library is missing
the product raises.

Every function restates, in eager fp32 PyTorch / numpy on the CPU, the algorithm
of one reference function, cited as ``file:line`` relative to the reference tree:

* ``neighbor_mask``        - src/tiled_swa.py:701-713 (window / neighbour sets)
* ``tiled_swa_ref``        - src/tiled_swa.py:693-717 (masked SDPA, additive 0/-1e6 mask)
* ``tiled_swa_explicit``   - same result via an explicit -inf masked softmax (independent path)
* ``tiled_swa_bruteforce`` - pure-Python loops over (query, key) pairs, tiny inputs only
* ``encode_idx``           - src/fused_rope2d.py:173-183
* ``decode_idx``/``pe_mask`` - src/fused_rope2d.py:40-45 and :212-219
* ``rope2d_ref``           - src/fused_rope2d.py:204-225
* ``rope2d_bwd_ref``       - src/fused_rope2d.py:110-122 (transposed rotation)
* ``flash_ref``            - src/flash_attn.py:625 (plain SDPA with scale)
* ``rope_tables``          - src/fused_rope2d.py:236-246: the self-test's table construction
                             (theta_i = base ** (-2 i / R), outer product with the positions,
                             cos and sin stacked on the last axis: [max_len, R, 2]).  The file
                             the module imports its tables from (src/rope2d.py) is absent from the
                             reference; this construction is the only one the reference holds.
                             Pinned in tests/test_oracle.py against the literal torch expression
                             of those lines and against unit-circle / angle-addition identities.
* ``swa_pairs``/``attn_flops`` - src/flash_attn.py:608-614 FLOP convention.
* ``tokens_to_image``/``image_to_tokens`` - src/tiled_swa.py:753-755 (tile-major [B, H, N, D] to the
                             image layout [B, IH, IW, H, D] and back); ``image_token_index`` is the
                             same map as a closed form, pinned against it and against loops.

Pinning status: the reference holds no golden vectors for this path.  Each
function above is pinned in ``tests/test_oracle.py`` by closed forms (neighbour
counts ``T(2W+1)-W(W+1)``), by brute force on tiny inputs, by reduction to library
routines (dense SDPA when the window covers the grid) and by invariants (row sums
of P, rotation orthogonality, identity on no-PE tokens).
"""
from __future__ import annotations

import math

import numpy as np
import torch
import torch.nn.functional as F

MASK_VALUE = -1e6  # src/tiled_swa.py:712 uses an additive -1e6, not -inf


# ------------------------------------------------------------------ layout adapters
def tokens_to_image(x: torch.Tensor, t_height: int, t_width: int, bh: int, bw: int) -> torch.Tensor:
    """[B, H, N, D] in tile-major token order -> image [B, t_height*bh, t_width*bw, H, D].

    src/tiled_swa.py:753-755: reshape to (B, H, TH, TW, BH, BW, D), permute (0, 2, 4, 3, 5, 1, 6),
    reshape to (B, TH*BH, TW*BW, H, D).
    """
    B, H, N, D = x.shape
    assert N == t_height * t_width * bh * bw
    return (x.reshape(B, H, t_height, t_width, bh, bw, D).permute(0, 2, 4, 3, 5, 1, 6)
            .reshape(B, t_height * bh, t_width * bw, H, D))


def image_to_tokens(x: torch.Tensor, t_height: int, t_width: int, bh: int, bw: int) -> torch.Tensor:
    """Inverse of ``tokens_to_image``: image [B, IH, IW, H, D] -> [B, H, N, D]."""
    B, IH, IW, H, D = x.shape
    assert IH == t_height * bh and IW == t_width * bw
    return (x.reshape(B, t_height, bh, t_width, bw, H, D).permute(0, 5, 1, 3, 2, 4, 6)
            .reshape(B, H, t_height * t_width * bh * bw, D))


def image_token_index(t_height: int, t_width: int, bh: int, bw: int) -> np.ndarray:
    """int64 [IH, IW]: token number of every pixel, n = ((y//bh * TW + x//bw) * bh + y%bh) * bw + x%bw."""
    y = np.arange(t_height * bh, dtype=np.int64)[:, None]
    x = np.arange(t_width * bw, dtype=np.int64)[None, :]
    return ((y // bh * t_width + x // bw) * bh + y % bh) * bw + x % bw


def image_token_offsets(t_height: int, t_width: int, bh: int, bw: int, stride_y: int, stride_x: int) -> np.ndarray:
    """int64 [N]: offset y * stride_y + x * stride_x of the pixel (y, x) that holds token n."""
    idx = image_token_index(t_height, t_width, bh, bw)
    out = np.empty(idx.size, dtype=np.int64)
    yy, xx = np.meshgrid(np.arange(idx.shape[0], dtype=np.int64), np.arange(idx.shape[1], dtype=np.int64), indexing="ij")
    out[idx.reshape(-1)] = (yy * stride_y + xx * stride_x).reshape(-1)
    return out


# --------------------------------------------------------------------------- a1
def neighbor_mask(t_height: int, t_width: int, row_size: int, col_size: int) -> np.ndarray:
    """bool [n_tiles, n_tiles]; entry (i, j) is True iff query tile i attends kv tile j.

    src/tiled_swa.py:701-713: tile (r, c) sees (r', c') iff |r-r'| <= row_size and
    |c-c'| <= col_size; the window is truncated at the grid border (never shifted).
    Tiles are numbered row-major (i = r * t_width + c).
    """
    r = np.arange(t_height)
    c = np.arange(t_width)
    row_ok = (r[None, :] >= r[:, None] - row_size) & (r[None, :] <= r[:, None] + row_size)
    col_ok = (c[None, :] >= c[:, None] - col_size) & (c[None, :] <= c[:, None] + col_size)
    total = row_ok[:, None, :, None] & col_ok[None, :, None, :]
    n = t_height * t_width
    return total.reshape(n, n)


def token_mask(b_size: int, t_height: int, t_width: int, row_size: int, col_size: int) -> np.ndarray:
    """bool [N, N] with N = n_tiles * b_size: every token of a tile shares the tile's set
    (src/tiled_swa.py:713)."""
    tm = neighbor_mask(t_height, t_width, row_size, col_size)
    n = tm.shape[0]
    return np.ascontiguousarray(np.broadcast_to(tm[:, None, :, None], (n, b_size, n, b_size))).reshape(n * b_size, n * b_size)


def axis_count(t: int, w: int) -> int:
    """Number of (i, j) pairs with |i-j| <= w on an axis of length t (closed form)."""
    w = min(w, t - 1)
    return t * (2 * w + 1) - w * (w + 1)


def swa_pairs(B: int, H: int, b_size: int, t_height: int, t_width: int, row_size: int, col_size: int) -> int:
    return B * H * b_size * b_size * axis_count(t_height, row_size) * axis_count(t_width, col_size)


def attn_flops(pairs: int, dk: int, dv: int) -> tuple[int, int]:
    """(forward, backward) FLOPs: fwd = QK^T + PV; bwd = S recompute, dV, dP, dK, dQ
    (the 2.5x convention of src/flash_attn.py:608-614 when dk == dv)."""
    return 2 * pairs * (dk + dv), 2 * pairs * (3 * dk + 2 * dv)


# --------------------------------------------------------------------------- a2
def tiled_swa_ref(q, k, v, b_size, t_height, t_width, row_size, col_size, sm_scale=1.0):
    """src/tiled_swa.py:693-717: SDPA with an additive 0 / -1e6 [N, N] mask."""
    B, H, N, _ = q.shape
    n_tiles = t_height * t_width
    assert N == n_tiles * b_size, "seqlen should match image size"
    allowed = torch.from_numpy(token_mask(b_size, t_height, t_width, row_size, col_size).copy())
    attn_mask = torch.where(allowed, 0.0, MASK_VALUE).to(q.dtype)
    return F.scaled_dot_product_attention(q, k, v, attn_mask=attn_mask, scale=sm_scale)


def tiled_swa_explicit(q, k, v, b_size, t_height, t_width, row_size, col_size, sm_scale=1.0,
                       return_lse2: bool = False):
    """Same operator written out: softmax over the allowed set only (-inf fill)."""
    allowed = torch.from_numpy(token_mask(b_size, t_height, t_width, row_size, col_size).copy())
    s = torch.matmul(q, k.transpose(-1, -2)) * sm_scale
    s = s.masked_fill(~allowed, float("-inf"))
    p = torch.softmax(s, dim=-1)
    o = torch.matmul(p, v)
    if return_lse2:
        # log2-domain log-sum-exp, the quantity the kernels save (src/tiled_swa.py:35,129)
        lse2 = torch.logsumexp(s, dim=-1) * (1.0 / math.log(2.0))
        return o, lse2
    return o


def tiled_swa_bruteforce(q, k, v, b_size, t_height, t_width, row_size, col_size, sm_scale=1.0):
    """Pure-Python loops; enumerates each query's neighbour tiles from the |dr|,|dc| rule
    without building a mask.  Tiny inputs only."""
    q = q.double().numpy(); k = k.double().numpy(); v = v.double().numpy()
    B, H, N, _ = q.shape
    o = np.zeros((B, H, N, v.shape[-1]))
    for b in range(B):
        for h in range(H):
            for r in range(t_height):
                for c in range(t_width):
                    keys = []
                    for r2 in range(max(r - row_size, 0), min(r + row_size, t_height - 1) + 1):
                        for c2 in range(max(c - col_size, 0), min(c + col_size, t_width - 1) + 1):
                            t2 = r2 * t_width + c2
                            keys.extend(range(t2 * b_size, (t2 + 1) * b_size))
                    keys = np.asarray(keys)
                    for s_ in range(b_size):
                        n = (r * t_width + c) * b_size + s_
                        logits = (k[b, h, keys] @ q[b, h, n]) * sm_scale
                        w = np.exp(logits - logits.max())
                        w /= w.sum()
                        o[b, h, n] = w @ v[b, h, keys]
    return torch.from_numpy(o)


def tiled_swa_grads(q, k, v, do, b_size, t_height, t_width, row_size, col_size, sm_scale=1.0,
                    fn=tiled_swa_ref):
    """(o, dq, dk, dv) by autograd through the eager expression (a3/a4 oracle)."""
    q = q.detach().clone().requires_grad_(True)
    k = k.detach().clone().requires_grad_(True)
    v = v.detach().clone().requires_grad_(True)
    o = fn(q, k, v, b_size, t_height, t_width, row_size, col_size, sm_scale)
    o.backward(do)
    return o.detach(), q.grad, k.grad, v.grad


def swa_delta(o, do):
    """delta = rowsum(o * do)  (src/tiled_swa.py:281)."""
    return (o.float() * do.float()).sum(-1)


# --------------------------------------------------------------------------- a5
def encode_idx(height: int, width: int) -> torch.Tensor:
    """src/fused_rope2d.py:181-183: idx = (row << 16) | col, row-major, int32."""
    rows = torch.arange(0, height)
    cols = torch.arange(0, width)
    return torch.bitwise_or(rows[:, None] << 16, cols).flatten().to(torch.int32)


def decode_idx(idx) -> tuple[np.ndarray, np.ndarray]:
    """(row, col) as int16: row = int16(idx >> 16) (arithmetic shift), col = int16(idx & 0xFFFF)
    (src/fused_rope2d.py:41-42; the eager reference :212-213 gives the same 16-bit values)."""
    a = np.asarray(idx, dtype=np.int32)
    row = (a >> 16).astype(np.int16)
    col = (a & 0xFFFF).astype(np.uint16).view(np.int16) if a.ndim else np.int16(np.uint16(a & 0xFFFF))
    return row, col


def pe_mask(idx) -> np.ndarray:
    """uint8 per token: bit0 = row axis rotated (row >= 0), bit1 = column axis rotated (col >= 0)
    (src/fused_rope2d.py:44-45, :216-219)."""
    row, col = decode_idx(idx)
    return ((row >= 0).astype(np.uint8) | ((col >= 0).astype(np.uint8) << 1)).astype(np.uint8)


# --------------------------------------------------------------------------- a6
def _cs_for(idx_axis: torch.Tensor, table: torch.Tensor):
    ok = (idx_axis >= 0)[:, None]
    safe = idx_axis.clamp(min=0).long()
    cos = torch.where(ok, table[safe, :, 0], torch.ones(()))
    sin = torch.where(ok, table[safe, :, 1], torch.zeros(()))
    return cos[None], sin[None]


def rope2d_ref(x, idx, cs_row_buffer, cs_col_buffer, inverse: bool = False):
    """src/fused_rope2d.py:204-225.  x [B', N, C]; returns a NEW tensor in x.dtype, math in fp32.

    dims [0,R) pair with [R,2R) (row angle), [2R,3R) with [3R,4R) (column angle), the rest
    passes through; an axis whose 16-bit index is negative is left unrotated (cos=1, sin=0).
    ``inverse`` applies the transposed rotation (src/fused_rope2d.py:114-115,121-122).
    """
    R = cs_row_buffer.shape[1]
    xf = x.float()
    row, col = decode_idx(idx.cpu().numpy())
    rc, rs = _cs_for(torch.from_numpy(row.astype(np.int64)), cs_row_buffer.float())
    cc, cs = _cs_for(torch.from_numpy(col.astype(np.int64)), cs_col_buffer.float())
    if inverse:
        rs, cs = -rs, -cs
    rx0, rx1 = xf[..., 0:R], xf[..., R:2 * R]
    cx0, cx1 = xf[..., 2 * R:3 * R], xf[..., 3 * R:4 * R]
    out = torch.cat([rx0 * rc - rx1 * rs, rx0 * rs + rx1 * rc,
                     cx0 * cc - cx1 * cs, cx0 * cs + cx1 * cc, xf[..., 4 * R:]], dim=-1)
    return out.to(x.dtype)


def rope2d_bwd_ref(do, idx, cs_row_buffer, cs_col_buffer):
    return rope2d_ref(do, idx, cs_row_buffer, cs_col_buffer, inverse=True)


# --------------------------------------------------------------------------- a7
def rope_tables(n_rdim: int, max_len: int, base: float = 10000.0) -> torch.Tensor:
    """[max_len, n_rdim, 2] fp32, (cos, sin) on the last axis (packing per
    src/fused_rope2d.py:236-240): theta_i = base ** (-2 i / n_rdim), entry [p, i] = exp(1j p theta_i).
    Evaluated in float64 as a complex exponential and rounded once to fp32."""
    theta = np.exp(-2.0 * np.log(float(base)) * np.arange(n_rdim, dtype=np.float64) / n_rdim)
    z = np.exp(1j * np.arange(max_len, dtype=np.float64)[:, None] * theta[None, :])
    return torch.from_numpy(np.stack([z.real, z.imag], axis=-1).astype(np.float32))


# --------------------------------------------------------------------------- a9/a10
def flash_ref(q, k, v, causal: bool, sm_scale: float):
    """src/flash_attn.py:625: plain SDPA; works for Lq != Lk and dk != dv."""
    return F.scaled_dot_product_attention(q, k, v, is_causal=causal, scale=sm_scale)


def flash_grads(q, k, v, do, causal, sm_scale):
    q = q.detach().clone().requires_grad_(True)
    k = k.detach().clone().requires_grad_(True)
    v = v.detach().clone().requires_grad_(True)
    o = flash_ref(q, k, v, causal, sm_scale)
    o.backward(do)
    return o.detach(), q.grad, k.grad, v.grad


def flash_lse2(q, k, sm_scale, causal: bool = False):
    """log2-domain log-sum-exp of the scaled scores, the vector M the forward pass saves
    (src/flash_attn.py:168-171: m_i + log2(l_i)); causal: keys up to the query's own index."""
    s = torch.matmul(q.float(), k.float().transpose(-1, -2)) * sm_scale
    if causal:
        Lq, Lk = s.shape[-2:]
        s = s.masked_fill(torch.arange(Lk)[None, :] > torch.arange(Lq)[:, None], float("-inf"))
    return torch.logsumexp(s, dim=-1) * (1.0 / math.log(2.0))


# --------------------------------------------------------------------------- composition (call stack 5)
def rope_swa_ref(q, k, v, idx, cs_row, cs_col, b_size, t_height, t_width, row_size, col_size, sm_scale):
    """RoPE on q and k, then SWA: the composition a fused kernel must equal."""
    B, H, N, C = q.shape
    qr = rope2d_ref(q.reshape(-1, N, C), idx, cs_row, cs_col).reshape(q.shape)
    kr = rope2d_ref(k.reshape(-1, N, C), idx, cs_row, cs_col).reshape(k.shape)
    return tiled_swa_ref(qr, kr, v, b_size, t_height, t_width, row_size, col_size, sm_scale)


def rope_swa_grads(q, k, v, do, idx, cs_row, cs_col, b_size, t_height, t_width, row_size, col_size, sm_scale):
    """(o, dq, dk, dv) w.r.t. the PRE-rotation q, k: dq_pre = R^T dq_post."""
    B, H, N, C = q.shape
    qr = rope2d_ref(q.reshape(-1, N, C), idx, cs_row, cs_col).reshape(q.shape)
    kr = rope2d_ref(k.reshape(-1, N, C), idx, cs_row, cs_col).reshape(k.shape)
    o, dqr, dkr, dv = tiled_swa_grads(qr, kr, v, do, b_size, t_height, t_width, row_size, col_size, sm_scale)
    dq = rope2d_bwd_ref(dqr.reshape(-1, N, C), idx, cs_row, cs_col).reshape(q.shape)
    dk = rope2d_bwd_ref(dkr.reshape(-1, N, C), idx, cs_row, cs_col).reshape(k.shape)
    return o, dq, dk, dv


# --------------------------------------------------------------------------- seeded inputs
def make_qkv(seed: int, B: int, H: int, Nq: int, Nk: int, dk: int, dv: int, dtype=torch.float32):
    """fp32 N(0,1) draws on the CPU from ``seed`` (q, k, v, do in that order), cast to dtype."""
    g = torch.Generator().manual_seed(seed)
    q = torch.randn((B, H, Nq, dk), generator=g)
    k = torch.randn((B, H, Nk, dk), generator=g)
    v = torch.randn((B, H, Nk, dv), generator=g)
    do = torch.randn((B, H, Nq, dv), generator=g)
    return tuple(t.to(dtype) for t in (q, k, v, do))


def make_rope_idx(seed: int, height: int, width: int, nope_frac: float = 0.05) -> torch.Tensor:
    """encode_idx(height, width) with a seeded ``nope_frac`` of tokens set to -1 (no-PE)."""
    g = torch.Generator().manual_seed(seed)
    idx = encode_idx(height, width).clone()
    if nope_frac > 0:
        idx[torch.rand(idx.shape[0], generator=g) < nope_frac] = -1
    return idx


def bf16_ulp_diff(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """|a - b| in units of bf16 ulps, on the ordered-integer representation of the bit patterns."""
    def key(t):
        i = t.to(torch.bfloat16).view(torch.int16).to(torch.int32)
        return torch.where(i < 0, -(i & 0x7FFF), i)
    return (key(a) - key(b)).abs()
