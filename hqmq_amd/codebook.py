"""Host-side algebra helpers with the reference's names.

`_make_24cell_codebook` mirrors src/quantizers/spherical.py:22-43 of the
reference (same vertex order: it defines the primary index p), `quat_mul`
mirrors src/quantizers/hqmq.py:33-41.  They are tiny torch functions used for
construction and inspection; the hot path computes the joint table on the GPU
(hqmq_build_joint).
"""
from __future__ import annotations

import torch


def _make_24cell_codebook(dtype=torch.float32) -> torch.Tensor:
    """(24, 4) Hurwitz units: p < 8 -> axis p//2 with sign (+ for even p); p >= 8 -> (+-1/2)^4,
    component j negative iff bit (3 - j) of p - 8 is set."""
    t = torch.zeros(24, 4, dtype=torch.float64)
    for p in range(8):
        t[p, p >> 1] = -1.0 if p & 1 else 1.0
    for m in range(16):
        for j in range(4):
            t[8 + m, j] = -0.5 if (m >> (3 - j)) & 1 else 0.5
    t = t.to(dtype)
    assert t.shape == (24, 4)
    return t


def quat_mul(q1: torch.Tensor, q2: torch.Tensor) -> torch.Tensor:
    """Hamilton product of (..., 4) tensors in (w, x, y, z) order."""
    a0, a1, a2, a3 = q1.unbind(dim=-1)
    b0, b1, b2, b3 = q2.unbind(dim=-1)
    return torch.stack((
        a0 * b0 - a1 * b1 - a2 * b2 - a3 * b3,
        a0 * b1 + a1 * b0 + a2 * b3 - a3 * b2,
        a0 * b2 - a1 * b3 + a2 * b0 + a3 * b1,
        a0 * b3 + a1 * b2 - a2 * b1 + a3 * b0,
    ), dim=-1)
