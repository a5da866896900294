"""Writes the small fixtures under tests/golden/ from the CPU oracle (run from the repo root:
``python tests/golden/make_golden.py``).  The reference ships no vectors for this path; these
files freeze the oracle's own outputs on seeded inputs so that a later change to the oracle
(or to PyTorch's SDPA) is noticed.  Inputs are regenerated from the seed, outputs are stored.
"""
import math
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import attn_oracle as orc  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def main():
    seed = 1234
    q, k, v, _ = orc.make_qkv(seed, 1, 2, 256, 256, 32, 32)
    o = orc.tiled_swa_ref(q, k, v, 1, 16, 16, 3, 3, 1 / math.sqrt(32))
    np.savez_compressed(os.path.join(HERE, "c1_swa_fwd.npz"), seed=seed, q=q.numpy(), v=v.numpy(), o=o.numpy())

    g = torch.Generator().manual_seed(77)
    x = torch.randn(2, 256, 24, generator=g)
    idx = orc.make_rope_idx(78, 16, 16, 0.1)
    idx[5] = (5 << 16) | 0xFFFF
    idx[6] = (-1 << 16) | 6
    y = orc.rope2d_ref(x, idx, orc.rope_tables(4, 16), orc.rope_tables(4, 16))
    np.savez_compressed(os.path.join(HERE, "rope_16x16.npz"), x=x.numpy(), idx=idx.numpy(), y=y.numpy(),
                        pe_bits=orc.pe_mask(idx.numpy()))


if __name__ == "__main__":
    main()
