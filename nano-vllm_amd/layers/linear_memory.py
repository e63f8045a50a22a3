"""Recurrent mixers with a decayed outer-product memory per head and per-sequence state slots, backed by gfx950 HIP
kernels.

``TokenShiftMix``: several blends of every row with the row before it, h + (h_prev - h) * mu_s, the last row of each
sequence carried in ``state[slot]``.  ``DecayMemory``: S <- diag(w) S + k v^T with w = exp(-exp(w_raw + w_bias)) per head
and key channel, read BEFORE the write as (S + diag(bonus) k v^T)^T r, normalised per head and gated by SiLU.
``ConvBiasSilu``: a short causal convolution with bias, then SiLU.  ``StateSpaceScan``: S <- a S + dt B x^T with one
scalar decay a = exp(-exp(A_log) dt) per head and step, dt = softplus(dt_raw + dt_bias), read AFTER the write as
S^T C + D x, times silu(z), in float32; ``group_rms_norm`` follows it.

The states [H, Dk, Dv] live in float32 in ``state[slot]``.  A slot is a row of the state tensors; the step's
``CacheContext.state_slots`` names the slot of every sequence of the batch.  A sequence whose rows start at position 0
starts from zero whatever its slot held before, so slots need no clearing.  The modules own no state: it is passed in.
"""
from __future__ import annotations

import torch
import torch.nn as nn

from .. import ops
from ..utils.cache_context import get_context

group_rms_norm = ops.group_rms_norm


class TokenShiftMix(nn.Module):
    def __init__(self, n_mix: int, channels: int, device=None):
        super().__init__()
        self.mu = nn.Parameter(torch.zeros(n_mix, channels, dtype=torch.float32, device=device))

    def forward(self, h: torch.Tensor, state: torch.Tensor) -> torch.Tensor:
        """h [T, C]; state [slots, C] of h's dtype; returns [n_mix, T, C]."""
        ctx = get_context()
        return ops.token_shift_mix(h, self.mu, state, ctx.cu_seqlens_q, ctx.cu_seqlens_k, ctx.state_slots)


class DecayMemory(nn.Module):
    def __init__(self, num_heads: int, key_dim: int, value_dim: int, eps: float, device=None):
        super().__init__()
        self.num_heads, self.key_dim, self.value_dim, self.eps = num_heads, key_dim, value_dim, eps
        f32 = dict(dtype=torch.float32, device=device)
        self.w_bias = nn.Parameter(torch.zeros(num_heads * key_dim, **f32))
        self.bonus = nn.Parameter(torch.zeros(num_heads, key_dim, **f32))
        self.norm_weight = nn.Parameter(torch.ones(num_heads * value_dim, **f32))

    def forward(self, r, k, v, w_raw, gate_raw, state: torch.Tensor) -> torch.Tensor:
        """r, k: [T, H, Dk]; v: [T, H, Dv]; w_raw [T, H * Dk], gate_raw [T, H * Dv] as projected; state
        [slots, H, Dk, Dv] float32.  Returns [T, H * Dv]."""
        ctx = get_context()
        return ops.decay_memory(r, k, v, w_raw, gate_raw, self.w_bias, self.bonus, self.norm_weight, state,
                                ctx.cu_seqlens_q, ctx.cu_seqlens_k, ctx.state_slots, self.eps)


class ConvBiasSilu(nn.Module):
    def __init__(self, channels: int, taps: int, device=None):
        super().__init__()
        self.channels, self.taps = channels, taps
        self.weight = nn.Parameter(torch.zeros(channels, taps, dtype=torch.float32, device=device))
        self.bias = nn.Parameter(torch.zeros(channels, dtype=torch.float32, device=device))

    def forward(self, x: torch.Tensor, conv_state: torch.Tensor) -> torch.Tensor:
        ctx = get_context()
        return ops.causal_conv_bias_silu(x, self.weight, self.bias, conv_state, ctx.cu_seqlens_q, ctx.cu_seqlens_k,
                                         ctx.state_slots)


class StateSpaceScan(nn.Module):
    def __init__(self, num_heads: int, groups: int, state_dim: int, head_dim: int, device=None):
        super().__init__()
        assert num_heads % groups == 0
        self.num_heads, self.groups, self.state_dim, self.head_dim = num_heads, groups, state_dim, head_dim
        f32 = dict(dtype=torch.float32, device=device)
        self.dt_bias = nn.Parameter(torch.zeros(num_heads, **f32))
        self.A_log = nn.Parameter(torch.zeros(num_heads, **f32))
        self.D = nn.Parameter(torch.zeros(num_heads, **f32))

    def forward(self, x, B, C, dt_raw, z, state: torch.Tensor) -> torch.Tensor:
        """x: [T, H, P]; B, C: [T, G, N]; dt_raw [T, H]; z [T, H * P]; state [slots, H, N, P] float32.
        Returns y * silu(z), float32 [T, H * P]."""
        ctx = get_context()
        return ops.state_space_scan(x, B, C, dt_raw, z, self.dt_bias, self.A_log, self.D, state, ctx.cu_seqlens_q,
                                    ctx.cu_seqlens_k, ctx.state_slots)
