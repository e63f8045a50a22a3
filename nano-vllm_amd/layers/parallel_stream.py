"""Layers around an fp32 residual stream that every layer reads through TWO RMS norms (one per parallel sublayer), backed
by gfx950 HIP kernels.

``HashedBigramEmbedding``: token embedding plus a row of a bigram table picked by a hash of (previous token, token)
(the table's extra last row at position 0), RMS-normed into the float32 stream; each sequence's last token id is
carried in ``prev_state[slot]``.  ``stream_boundary_pair``: everything that happens to the stream between two layers in
ONE launch: the sublayers' outputs are added (matmul-dtype tensors, fp32 parts such as the outputs of the chosen
experts times a common weight, and outputs that are RMS-normed on their way in), and up to two norms of the result are
written side by side in float32 for the next layer's sublayers.  ``ReluSquared``: max(x, 0)^2.
"""
from __future__ import annotations

import torch
import torch.nn as nn

from .. import ops
from ..utils.cache_context import get_context

stream_boundary_pair = ops.stream_boundary_pair


class HashedBigramEmbedding(nn.Module):
    def __init__(self, vocab: int, width: int, buckets: int, mul_prev: int, mul_cur: int, eps: float, dtype=None,
                 device=None, normed: bool = True):
        """buckets = 0: no bigram table (the embedding row alone is normed).  normed=False: the sum of the rows goes
        into the stream as it is."""
        super().__init__()
        self.buckets, self.mul_prev, self.mul_cur, self.eps = int(buckets), int(mul_prev), int(mul_cur), float(eps)
        self.weight = nn.Parameter(torch.zeros(vocab, width, dtype=dtype, device=device))
        self.bigram = nn.Parameter(torch.zeros(buckets + 1, width, dtype=dtype, device=device)) if buckets else None
        self.norm = nn.Parameter(torch.ones(width, dtype=torch.float32, device=device)) if normed else None

    def forward(self, ids: torch.Tensor, positions: torch.Tensor, prev_state: torch.Tensor | None) -> torch.Tensor:
        """ids, positions [T] int64; prev_state [slots] int64; returns the stream [T, W] float32."""
        ctx = get_context()
        return ops.hashed_bigram_embed(ids, positions, self.weight, self.bigram, self.mul_prev, self.mul_cur, self.norm,
                                       self.eps, prev_state, ctx.cu_seqlens_q, ctx.state_slots)


class ReluSquared(nn.Module):
    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return ops.relu_squared(x)
