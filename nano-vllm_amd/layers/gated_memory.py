"""Recurrent mixers whose memory is written before it is read, with per-sequence state slots, backed by gfx950 HIP
kernels.

``MatrixLSTMMemory``: per head a matrix memory S [Dk, Dv] with exponential input and forget gates, a normaliser vector n
and a running maximum m that keeps the exponentials bounded (m starts at 0):
    m' = max(f + m, i);  S <- exp(f + m - m') S + exp(i - m') k v^T;  n likewise with k;  o = S^T q / (max(|n . q|, exp(-m')) + 1e-6)
with i = cap tanh((i_pre + b_i) / cap) and f = logsigmoid(cap tanh((f_pre + b_f) / cap)); the read-out is normalised per
head, weighted and gated by a sigmoid.  ``GatedWriteMemory``: S <- diag(f) S + (1 - f) v^T, o = S^T silu(q), with
f = lower + (1 - lower) sigmoid(f_raw + b_f) per head and key channel; the read-out is normalised per head with one
weight [Dv] for all heads.

States live in float32 in ``state[slot]`` tensors that the caller passes in; a sequence whose rows start at position 0
starts from zeros whatever its slot held before, so slots need no clearing.
"""
from __future__ import annotations

import torch
import torch.nn as nn

from .. import ops
from ..utils.cache_context import get_context


class MatrixLSTMMemory(nn.Module):
    def __init__(self, num_heads: int, key_dim: int, value_dim: int, gate_cap: float, eps: float, device=None):
        super().__init__()
        self.num_heads, self.key_dim, self.value_dim = num_heads, key_dim, value_dim
        self.gate_cap, self.eps, self.q_scale = float(gate_cap), float(eps), float(key_dim) ** -0.5
        f32 = dict(dtype=torch.float32, device=device)
        self.i_bias = nn.Parameter(torch.zeros(num_heads, **f32))
        self.f_bias = nn.Parameter(torch.zeros(num_heads, **f32))
        self.norm_weight = nn.Parameter(torch.ones(num_heads * value_dim, **f32))

    def state_shapes(self) -> dict:
        H, Dk, Dv = self.num_heads, self.key_dim, self.value_dim
        return {"state": ((H, Dk, Dv), torch.float32), "normaliser": ((H, Dk), torch.float32), "maximum": ((H,), torch.float32)}

    def forward(self, q, k, v, gates_pre, gate_raw, cache: dict) -> torch.Tensor:
        """q, k: [T, H, Dk]; v: [T, H, Dv]; gates_pre [T, 2 H] float32 (input gates, then forget gates, no bias);
        gate_raw [T, H * Dv]; cache: the tensors of `state_shapes()` with a leading slot dimension.  Returns [T, H * Dv]."""
        ctx = get_context()
        return ops.mlstm_memory(q, k, v, gates_pre, gate_raw, self.i_bias, self.f_bias, self.norm_weight, cache["state"],
                                cache["normaliser"], cache["maximum"], ctx.cu_seqlens_q, ctx.cu_seqlens_k, ctx.state_slots,
                                self.eps, self.gate_cap, self.q_scale)


class GatedWriteMemory(nn.Module):
    def __init__(self, num_heads: int, key_dim: int, value_dim: int, eps: float, device=None):
        super().__init__()
        self.num_heads, self.key_dim, self.value_dim, self.eps = num_heads, key_dim, value_dim, float(eps)
        f32 = dict(dtype=torch.float32, device=device)
        self.f_bias = nn.Parameter(torch.zeros(num_heads * key_dim, **f32))
        self.lower = nn.Parameter(torch.zeros(num_heads * key_dim, **f32))
        self.norm_weight = nn.Parameter(torch.ones(value_dim, **f32))

    def state_shapes(self) -> dict:
        return {"state": ((self.num_heads, self.key_dim, self.value_dim), torch.float32)}

    def forward(self, q, f_raw, v, cache: dict) -> torch.Tensor:
        """q, f_raw: [T, H, Dk] as projected; v: [T, H, Dv]; returns [T, H * Dv]."""
        ctx = get_context()
        return ops.gated_write_memory(q, f_raw, v, self.f_bias, self.lower, self.norm_weight, cache["state"],
                                      ctx.cu_seqlens_q, ctx.cu_seqlens_k, ctx.state_slots, self.eps)
