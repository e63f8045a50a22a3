"""Routed experts (mixture of experts), backed by gfx950 HIP kernels: top-k routing with a softmax over the chosen
logits, the (token, choice) pairs sorted by expert on the device, and both expert products as grouped MFMA matrix
products over row tiles of one expert each (no host round trip, no atomics).

Expert: g = min(G h, limit), u = clamp(U h, -limit, limit), D (g * sigmoid(alpha g) * (u + 1)); no biases.

``TableExperts``: no router; a table [vocab, top] names the experts of every token id, the expert is the plain SiLU-gated
unit D (silu(G h) * (U h)), and the caller weights the outputs (each expert counts 1 / top).
"""
from __future__ import annotations

import torch
import torch.nn as nn

from .. import ops


class MoEExperts(nn.Module):
    def __init__(self, top: int, limit: float, alpha: float = 1.702):
        super().__init__()
        self.top, self.limit, self.alpha = int(top), float(limit), float(alpha)

    def forward(self, h: torch.Tensor, logits: torch.Tensor, gate_up: torch.Tensor, down: torch.Tensor) -> torch.Tensor:
        """h [T, W]; logits [T, E] float32; gate_up [E, 2 ff, W] (gate rows, then up rows); down [E, W, ff].
        Returns the weighted expert outputs [T, top, W] float32."""
        return ops.moe_experts(h, logits, gate_up, down, self.top, self.limit, self.alpha)


class TableExperts(nn.Module):
    def __init__(self, top: int):
        super().__init__()
        self.top = int(top)

    def forward(self, h: torch.Tensor, table: torch.Tensor, token_ids: torch.Tensor, gate_up: torch.Tensor,
                down: torch.Tensor) -> torch.Tensor:
        """h [T, W]; table [vocab, top] int32; token_ids [T] int64; gate_up [E, 2 ff, W]; down [E, W, ff].
        Returns the unweighted expert outputs [T, top, W] float32."""
        return ops.moe_table_experts(h, table[token_ids].contiguous(), gate_up, down)
