"""Rotary position encoding, half-split layout."""

from __future__ import annotations

import torch

from tokamak_amd.config.registry import register_part
from tokamak_amd.kernels import ops
from tokamak_amd.parts.base import PositionData, PositionEncoding


class RotaryHalf(PositionEncoding):
    """cos/sin tables for a step's positions.

    inv_freq[j] = 1 / theta^(2j / rotary_dim), float32, computed on the host
    exactly as written in reference: src/tokamak/model/layers.py:47; the angle
    float(pos) * inv_freq[j] and its cos/sin are float32 (layers.py:56-58).  The
    rotation itself pairs dim j with dim j + rotary_dim/2 (layers.py:61-63) and
    is applied by the mixer's fused kernel.
    """

    capturable = True
    replayable = True

    def __init__(self, *, rotary_dim: int, theta: float, dtype, device) -> None:
        super().__init__(dtype=dtype, device=device)
        if rotary_dim % 2:
            raise ValueError(f"rotary_dim must be even, got {rotary_dim}")
        self.rotary_dim = int(rotary_dim)
        self.theta = float(theta)
        inv_freq = 1.0 / (self.theta ** (torch.arange(0, rotary_dim, 2, dtype=torch.float32) / rotary_dim))
        self.inv_freq = inv_freq.to(self.device)
        self.key = ("rotary_half", self.rotary_dim, self.theta)

    def prepare(self, batch) -> PositionData:
        """cos and sin, each float32 [N, rotary_dim/2]; computed once per step."""
        cached = batch.memo.get(self.key)
        if cached is None:
            n, half = batch.num_tokens, self.rotary_dim // 2
            cos = torch.empty((n, half), dtype=torch.float32, device=self.device)
            sin = torch.empty((n, half), dtype=torch.float32, device=self.device)
            ops.rope_tables(batch.positions, self.inv_freq, cos, sin)
            cached = batch.memo[self.key] = PositionData(cos=cos, sin=sin, rotary_dim=self.rotary_dim)
        return cached


register_part("position", "rotary_half", RotaryHalf)
