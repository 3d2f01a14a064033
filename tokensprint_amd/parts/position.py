"""Rotate-half rotary position encoding.

Table as the reference's table variant builds it (engine/nn/rope.py:28-29,105-109):
inv_freq[i] = 1/theta^(2i/dim) in float32, angle = float32(pos) * inv_freq, then
cos and sin; the pairing (x[i], x[i+dim/2]) is engine/kernels/triton/rope.py:53-65.
The table is computed on the host so every device run reads identical values.
"""

from __future__ import annotations

import torch

from tokensprint_amd.parts.base import POSITIONS, PositionEncoding, register


@register(POSITIONS, "rope")
class RotaryEncoding(PositionEncoding):
    """params: dim (rotated head size), theta, max_position."""

    def __init__(self, params, ctx):
        super().__init__(params, ctx)
        self.dim = int(params["dim"])
        self.theta = float(params["theta"])
        self.max_position = int(params["max_position"])
        if self.dim % 2:
            raise ValueError(f"rotary dim must be even, got {self.dim}")
        idx = torch.arange(0, self.dim, 2, dtype=torch.float32)
        inv_freq = 1.0 / (self.theta ** (idx / self.dim))
        angles = torch.outer(torch.arange(self.max_position, dtype=torch.float32), inv_freq)
        self.cos = angles.cos().contiguous().to(ctx.device)
        self.sin = angles.sin().contiguous().to(ctx.device)

    def rotary_tables(self):
        return self.cos, self.sin

    def step_read_tensors(self):
        return []          # a step reads the rows of its positions, not the tables

    def apply(self, q, k, positions):
        self.ops.rope_inplace(q, positions, self.cos, self.sin)
        if k is not None:
            self.ops.rope_inplace(k, positions, self.cos, self.sin)
