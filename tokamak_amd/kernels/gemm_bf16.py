"""bfloat16 matrix products with float32 accumulation."""

from __future__ import annotations

import torch

from tokamak_amd.kernels import ops


def gemm(x: torch.Tensor, weight: torch.Tensor, out: torch.Tensor) -> None:
    """out[M, N] = x[M, K] @ weight[N, K]^T; out is bfloat16 or float32."""
    if out.dtype == torch.bfloat16:
        torch.matmul(x, weight.t(), out=out)
    else:
        ops.gemm_tiled(x, weight, out)
