"""Sigmoid attention inside fixed chunks of positions with rotated values, over the paged KV cache, backed by gfx950 HIP
kernels.

Queries and keys are RMS-normed over their WHOLE projection (all heads at once, one weight per column) and rotated
(rotate-half pairs on the first rot_dims dimensions of every head); values are rotated over all their dimensions by
their own position and cached so.  Query i sees key j <= i of its own chunk, floor(i / chunk) == floor(j / chunk), with
the weight sigmoid(scale q.k + bias of the head), not normalised over keys; the weighted sum of the rotated values is
turned back by the query's position.  A step's rows may be prompt portions and single decoded tokens side by side:
portions go to the bf16 MFMA tile kernel where it is built for the head sizes, everything else to the one-wave-per-row
kernel.
"""
from __future__ import annotations

import numpy as np
import torch
import torch.nn as nn

from .. import ops
from ..utils.cache_context import get_context

TILE_ROWS = 64


def rotary_frequencies(dims: int, base: float) -> torch.Tensor:
    """base^(-2 i / dims) for i < dims / 2, computed in float64 and rounded once."""
    return torch.tensor([float(base) ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=torch.float32)


def query_tiles(ctx) -> tuple | None:
    """(tile_seq, tile_q0, has_single_rows) for the step: the rows of every sequence with several rows cut into blocks
    of TILE_ROWS; built once per step from the host copy of cu_seqlens_q and kept on the context.  None when the host
    copy is missing or no sequence has several rows."""
    cached = getattr(ctx, "_query_tiles", False)
    if cached is not False:
        return cached
    tiles = None
    cu = ctx.cu_seqlens_q_host
    if cu is not None and ctx.max_seqlen_q > 1:
        n = np.diff(cu)
        seqs, q0 = [], []
        for b in np.nonzero(n > 1)[0]:
            starts = np.arange(0, n[b], TILE_ROWS, dtype=np.int32)
            seqs.append(np.full(len(starts), b, dtype=np.int32))
            q0.append(starts)
        if seqs:
            dev = ctx.cu_seqlens_q.device
            tiles = (torch.from_numpy(np.concatenate(seqs)).to(dev), torch.from_numpy(np.concatenate(q0)).to(dev),
                     bool((n == 1).any()))
    ctx._query_tiles = tiles
    return tiles


class ChunkSigmoidAttention(nn.Module):
    def __init__(self, num_heads: int, num_kv_heads: int, head_dim: int, v_head_dim: int, scale: float, chunk: int,
                 rot_dims: int, rot_base: float, eps: float, device=None):
        super().__init__()
        assert num_heads % num_kv_heads == 0 and rot_dims % 2 == 0 and rot_dims <= head_dim and v_head_dim % 2 == 0
        self.num_heads, self.num_kv_heads, self.head_dim, self.v_head_dim = num_heads, num_kv_heads, head_dim, v_head_dim
        self.scale, self.chunk, self.rot_dims, self.eps = float(scale), int(chunk), int(rot_dims), float(eps)
        f32 = dict(dtype=torch.float32, device=device)
        self.q_norm = nn.Parameter(torch.ones(num_heads * head_dim, **f32))
        self.k_norm = nn.Parameter(torch.ones(num_kv_heads * head_dim, **f32))
        self.head_bias = nn.Parameter(torch.zeros(num_heads, **f32))
        self.register_buffer("freq", rotary_frequencies(rot_dims, rot_base).to(device) if rot_dims else None, persistent=False)
        self.register_buffer("value_freq", rotary_frequencies(v_head_dim, rot_base).to(device), persistent=False)

    def forward(self, q, k, v, positions, k_cache, v_cache) -> torch.Tensor:
        """q: [T, H, D]; k: [T, G, D]; v: [T, G, Dv] as projected; caches [num_blocks, block_size, G, D | Dv].
        Returns [T, H * Dv]."""
        ctx = get_context()
        qp = ops.chunk_attn_prep_store(positions, q, k, v, self.q_norm, self.k_norm, self.eps, self.freq, self.rot_dims,
                                       self.value_freq, ctx.slot_mapping, k_cache, v_cache)
        tiles = None
        if ops.chunk_sigmoid_tile_ok(self.head_dim, self.v_head_dim, q.dtype):
            tiles = query_tiles(ctx)
        return ops.attn_chunk_sigmoid_paged(qp, k_cache, v_cache, ctx.cu_seqlens_q, ctx.cu_seqlens_k, ctx.block_tables,
                                            self.scale, self.head_bias, self.chunk, self.value_freq,
                                            tiles[:2] if tiles else None, tiles[2] if tiles else True)
