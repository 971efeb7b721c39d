"""y = x @ W^T for the projections of a step.

float32: the hand-written tiled kernel (true 32-bit multiply-add, row-wise
deterministic).  bfloat16: hand-written MFMA kernels when the shape fits them,
else the library product that torch binds (as the reference's nn.Linear does).
"""

from __future__ import annotations

import torch

from tokamak_amd.kernels import ops


def linear(x: torch.Tensor, weight: torch.Tensor, out_dtype: torch.dtype | None = None) -> torch.Tensor:
    """``x`` [M, K], ``weight`` [N, K] -> [M, N] in ``out_dtype`` (default: x's)."""
    out_dtype = out_dtype or x.dtype
    m, n = x.shape[0], weight.shape[0]
    out = torch.empty((m, n), dtype=out_dtype, device=x.device)
    if m == 0:
        return out
    if x.dtype == torch.float32:
        ops.gemm_tiled(x, weight, out)
        return out
    from tokamak_amd.kernels import gemm_bf16

    gemm_bf16.gemm(x, weight, out)
    return out
