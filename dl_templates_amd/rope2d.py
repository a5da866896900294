"""cos/sin table holder for the 2D rotary encoding.

The reference imports ``FusedRotaryPositionEncodingContext`` from ``src/rope2d.py``
(src/fused_rope2d.py:8), a file that is not part of the reference tree.  Its contract is
recovered from the call sites: ``Context(n_components, max_len)`` exposes
``.cs_components`` of shape ``[max_len, n_rdim, 2]`` with (cos, sin) on the last axis
(src/fused_rope2d.py:22-23, :128, :193-194, :201 and the table built in the self-test,
:236-246).  ``n_components`` is the number of head dims one axis occupies, so
``n_rdim = n_components // 2`` rotation pairs.  The frequency schedule has the form of the only
table construction the reference holds, its self-test (src/fused_rope2d.py:236-240):
``theta_i = base ** (-2 i / n_rdim)``, position p turns pair i by ``p * theta_i``; the self-test
uses base 1000, the default here is 10000.  Angles are formed in float64 and rounded once to
fp32.  The kernels accept any table, so a caller who owns the original file keeps its values.
"""
from __future__ import annotations

import numpy as np
import torch


class FusedRotaryPositionEncodingContext(torch.nn.Module):
    def __init__(self, n_components: int, max_len: int, base: float = 10000.0):
        super().__init__()
        if n_components % 2 != 0:
            raise ValueError("n_components must be even (pairs of dims are rotated)")
        self.n_components = n_components
        self.n_rdim = n_components // 2
        self.max_len = max_len
        self.base = float(base)
        inv = np.power(self.base, -2.0 * np.arange(self.n_rdim, dtype=np.float64) / max(self.n_rdim, 1))
        ang = np.outer(np.arange(max_len, dtype=np.float64), inv)
        table = torch.from_numpy(np.stack([np.cos(ang), np.sin(ang)], axis=-1).astype(np.float32))
        self.register_buffer("cs_components", table, persistent=False)
