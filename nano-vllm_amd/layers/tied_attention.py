"""Causal softmax attention over the paged KV cache that reads its VALUES from its un-prepared keys, backed by gfx950
HIP kernels.

``ShortConv``: a short causal convolution over time per channel, no bias and no activation, the last taps - 1 inputs of
each sequence carried in ``state[slot]``.  ``KeyTiedAttention``: queries and keys are RMS-normed per head (one weight [D]
for all heads) and rotated on their first rot_dims dimensions (rotate-half pairs; the frequencies may be rescaled by
wavelength); the key cache holds the prepared keys, the value cache the keys as they came in; scores are
scale * q . k in float32, ordinary softmax over the visible keys.  The attention itself is the score-modified kernel
family with every modifier switched off.
"""
from __future__ import annotations

import torch
import torch.nn as nn

from .. import ops
from ..utils.cache_context import get_context
from .rope import llama3_scale_inv_freq


def scaled_rotary_frequencies(dims: int, base: float, scaling: dict | None = None) -> torch.Tensor:
    """base^(-2 i / dims) for i < dims / 2 in double precision; with `scaling` (factor, low, high, original) wavelengths
    above original / low are stretched by factor, those below original / high kept, the band between blended.  Rounded
    to float32 once."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = float(base) ** (-2.0 * i / dims)
    if scaling:
        f = llama3_scale_inv_freq(f, float(scaling["factor"]), float(scaling["low"]), float(scaling["high"]),
                                  float(scaling["original"]))
    return f.to(torch.float32)


class ShortConv(nn.Module):
    def __init__(self, channels: int, taps: int, device=None):
        super().__init__()
        self.channels, self.taps = channels, taps
        self.weight = nn.Parameter(torch.zeros(channels, taps, dtype=torch.float32, device=device))

    def forward(self, x: torch.Tensor, conv_state: torch.Tensor) -> torch.Tensor:
        ctx = get_context()
        return ops.causal_conv(x, self.weight, conv_state, ctx.cu_seqlens_q, ctx.cu_seqlens_k, ctx.state_slots)


class KeyTiedAttention(nn.Module):
    def __init__(self, num_heads: int, num_kv_heads: int, head_dim: int, scale: float, eps: float, rot_dims: int = 0,
                 rot_base: float = 10000.0, rot_scaling: dict | None = None, device=None):
        super().__init__()
        assert num_heads % num_kv_heads == 0 and rot_dims % 2 == 0 and rot_dims <= head_dim
        self.num_heads, self.num_kv_heads, self.head_dim = num_heads, num_kv_heads, head_dim
        self.scale, self.eps, self.rot_dims = float(scale), float(eps), int(rot_dims)
        f32 = dict(dtype=torch.float32, device=device)
        self.q_norm = nn.Parameter(torch.ones(head_dim, **f32))
        self.k_norm = nn.Parameter(torch.ones(head_dim, **f32))
        freq = scaled_rotary_frequencies(rot_dims, rot_base, rot_scaling) if rot_dims else None
        self.register_buffer("freq", freq.to(device) if freq is not None else None, persistent=False)

    def forward(self, q, k, positions, k_cache, v_cache) -> torch.Tensor:
        """q: [T, H, D]; k: [T, G, D]; caches [num_blocks, block_size, G, D].  Returns [T, H * D]."""
        ctx = get_context()
        qp = ops.head_norm_rope_store(positions, q, k, self.q_norm, self.k_norm, self.eps, self.freq, self.rot_dims,
                                      ctx.slot_mapping, k_cache, v_cache)
        singles = -1 if ctx.num_decode_seqs is None else int(ctx.num_decode_seqs > 0)
        return ops.attn_scoremod_paged(qp, k_cache, v_cache, ctx.cu_seqlens_q, ctx.cu_seqlens_k, ctx.block_tables,
                                       self.scale, 0.0, None, None, ctx.max_seqlen_q, ctx.max_seqlen_k, singles)
