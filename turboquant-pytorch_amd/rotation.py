"""
Random orthogonal rotation used by the codec.

Same recipe as the reference's generate_rotation_matrix (turboquant/turboquant.py:18-33):
a d x d standard Gaussian drawn from a CPU generator seeded with `seed`, QR-decomposed, and
the columns of Q multiplied by the signs of diag(R) (zero counts as +1) so that the
factorisation -- and therefore the matrix for a given seed -- is unique.  The matrix is
always produced on the host; rotated = x @ Pi.T, un-rotated = y @ Pi.
"""
from __future__ import annotations

from typing import Optional

import torch


def generate_rotation_matrix(d: int, seed: Optional[int] = None, device: str = "cpu") -> torch.Tensor:
    gen = torch.Generator(device="cpu")
    if seed is not None:
        gen.manual_seed(seed)
    gauss = torch.randn(d, d, generator=gen)
    q, r = torch.linalg.qr(gauss)
    signs = torch.where(torch.diagonal(r) < 0, -1.0, 1.0).to(q.dtype)
    return (q * signs.unsqueeze(0)).to(device)
