"""Routed experts (mixture of experts), backed by gfx950 HIP kernels: top-k routing with a softmax over the chosen
logits, the (token, choice) pairs sorted by expert on the device, and both expert products as grouped MFMA matrix
products over row tiles of one expert each (no host round trip, no atomics).

Expert: g = min(G h, limit), u = clamp(U h, -limit, limit), D (g * sigmoid(alpha g) * (u + 1)); no biases.

``TableExperts``: no router; a table [vocab, top] names the experts of every token id, the expert is the plain SiLU-gated
unit D (silu(G h) * (U h)), and the caller weights the outputs (each expert counts 1 / top).

``GroupedSigmoidRouter``: scores are sigmoids of the router logits; the choice is made on score + a per-expert
correction, among the experts of the best consecutive blocks of experts (a block's merit: the sum of its top two biased
scores); the weights are the plain scores of the chosen, used as they are.  ``SquaredReluExperts``: experts
without a gate, D max(U h, 0)^2, weighted by the router's weights.
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


class GroupedSigmoidRouter(nn.Module):
    def __init__(self, experts: int, top: int, groups: int = 1, keep_groups: int = 1, device=None):
        super().__init__()
        if experts % groups or not 1 <= keep_groups <= groups or not 1 <= top <= keep_groups * (experts // groups):
            raise ValueError("groups must divide the experts, and the kept groups must hold `top` experts")
        self.experts, self.top, self.groups, self.keep_groups = int(experts), int(top), int(groups), int(keep_groups)
        self.correction = nn.Parameter(torch.zeros(experts, dtype=torch.float32, device=device))

    def forward(self, logits: torch.Tensor) -> tuple:
        """logits [T, E] float32 -> (ids [T, top] int32, weights [T, top] float32)."""
        return ops.moe_route_grouped(logits, self.correction, self.top, self.groups, self.keep_groups)


class SquaredReluExperts(nn.Module):
    def forward(self, h: torch.Tensor, ids: torch.Tensor, weights: torch.Tensor, up: torch.Tensor,
                down: torch.Tensor) -> torch.Tensor:
        """h [T, W]; ids / weights [T, top]; up [E, ff, W]; down [E, W, ff].  Returns the weighted expert outputs
        [T, top, W] float32."""
        return ops.moe_relu2_experts(h, ids, weights, up, down)
