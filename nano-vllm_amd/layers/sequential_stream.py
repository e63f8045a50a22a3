"""Layers around a pre-norm fp32 residual stream whose sublayers run one after the other, backed by gfx950 HIP kernels.

``stream_boundary_scaled``: everything that happens to the stream between two sublayers in ONE launch: the sublayer's
output (a matmul-dtype tensor, a second one behind a per-row sigmoid gate such as a shared expert, fp32 parts such as
the weighted outputs of the chosen experts) is scaled per column and added, and the next sublayer's RMS norm of the
result is written in the matmul dtype and / or float32.  ``OnePlusNorm``: an RMS-norm weight stored as an offset from
one; the weight as applied is kept in float32.  ``PolyNorm``: a z / rms(z) + b z^2 / rms(z^2) + c z^3 / rms(z^3) + e per
row, powers element by element.
"""
from __future__ import annotations

import torch
import torch.nn as nn

from .. import ops

stream_boundary_scaled = ops.stream_boundary_scaled


class OnePlusNorm(nn.Module):
    """Holds the stored weight w; `applied` is 1 + w in float32 (refreshed by `finalize()` after loading)."""

    def __init__(self, width: int, device=None):
        super().__init__()
        self.weight = nn.Parameter(torch.zeros(width, dtype=torch.float32, device=device))
        self.register_buffer("applied", torch.ones(width, dtype=torch.float32, device=device), persistent=False)

    def finalize(self) -> None:
        self.applied = (1.0 + self.weight.data.float()).contiguous()


class PolyNorm(nn.Module):
    def __init__(self, eps: float, device=None):
        super().__init__()
        self.eps = float(eps)
        self.coef = nn.Parameter(torch.zeros(4, dtype=torch.float32, device=device))

    def forward(self, z: torch.Tensor) -> torch.Tensor:
        return ops.poly_norm(z, self.coef, self.eps)
