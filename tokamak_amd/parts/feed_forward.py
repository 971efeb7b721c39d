"""Feed-forward parts."""

from __future__ import annotations

import torch

from tokamak_amd.config.registry import register_part
from tokamak_amd.kernels.linear import gated_linear, linear
from tokamak_amd.parts.base import FeedForward, Fetch
from tokamak_amd.weights.spec import TensorSpec


class SwiGLU(FeedForward):
    """down(silu(gate(x)) * up(x)), no biases
    (reference: src/tokamak/model/layers.py:92-104).

    ``gate_proj`` and ``up_proj`` are held as one [2I, H] matrix so one product
    yields both halves.
    """

    capturable = True
    fuses_residual = True
    replayable = True

    def __init__(self, *, hidden_size: int, intermediate_size: int, dtype, device) -> None:
        super().__init__(dtype=dtype, device=device)
        self.hidden_size = int(hidden_size)
        self.intermediate_size = int(intermediate_size)
        self.gate_up: torch.Tensor | None = None
        self.down: torch.Tensor | None = None

    def expected_tensors(self, prefix: str) -> dict[str, TensorSpec]:
        h, i = self.hidden_size, self.intermediate_size
        return {
            prefix + "gate_proj.weight": TensorSpec((i, h)),
            prefix + "up_proj.weight": TensorSpec((i, h)),
            prefix + "down_proj.weight": TensorSpec((h, i)),
        }

    def bind(self, prefix: str, fetch: Fetch) -> None:
        self.gate_up = torch.cat([fetch(prefix + "gate_proj.weight"), fetch(prefix + "up_proj.weight")], dim=0).contiguous()
        self.down = fetch(prefix + "down_proj.weight")

    def forward(self, h, batch, add_into=None):
        return linear(gated_linear(h, self.gate_up), self.down, allow_partials=True, add_into=add_into)


register_part("feed_forward", "swiglu", SwiGLU)
