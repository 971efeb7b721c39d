"""RMSNorm fused with the residual add."""

from __future__ import annotations

import torch

from tokamak_amd.config.registry import register_part
from tokamak_amd.kernels import ops
from tokamak_amd.kernels.linear import Added, DeferredNorm, StreamSink
from tokamak_amd.parts.base import Fetch, Norm
from tokamak_amd.weights.spec import TensorSpec


class RMSNorm(Norm):
    """x = resid + delta; out = x * rsqrt(mean(x^2) + eps) * weight.

    Statistics and the product with the weight are float32; one rounding to the
    compute dtype at the end (reference: src/tokamak/model/layers.py:28-33
    computes the statistics in float32, rounds, then multiplies by the weight).
    """

    capturable = True
    fuses_residual = True
    replayable = True

    def __init__(self, *, dim: int, eps: float, dtype, device) -> None:
        super().__init__(dtype=dtype, device=device)
        self.dim = int(dim)
        self.eps = float(eps)
        self.weight: torch.Tensor | None = None

    def expected_tensors(self, prefix: str) -> dict[str, TensorSpec]:
        return {prefix + "weight": TensorSpec((self.dim,), role="vector")}

    def bind(self, prefix: str, fetch: Fetch) -> None:
        self.weight = fetch(prefix + "weight")

    def sink(self, resid: torch.Tensor) -> StreamSink:
        return StreamSink(resid, self.weight)

    def forward(self, resid, delta, *, rows=None, write_resid=True, defer=False):
        if isinstance(delta, Added):
            # the product before has added into the stream; if it has left the stream times
            # this norm's weight, the product after may finish the norm
            if defer and rows is None and delta.scaled is not None and delta.gamma is self.weight:
                return DeferredNorm(resid, self.weight, self.eps, self.dtype, delta.scaled, delta.sumsq)
            delta = None
        m = resid.shape[0] if rows is None else rows.numel()
        out = torch.empty((m, self.dim), dtype=self.dtype, device=resid.device)
        ops.add_rmsnorm(resid, delta, self.weight, self.eps, out, rows=rows, write_resid=write_resid)
        return out


register_part("norm", "rmsnorm", RMSNorm)
