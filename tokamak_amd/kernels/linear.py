"""y = x @ W^T for the projections of a step.

float32: the hand-written tiled kernel (true 32-bit multiply-add, row-wise
deterministic).  bfloat16: hand-written MFMA kernels for up to 64 rows, else
the library product that torch binds (as the reference's nn.Linear does).
"""

from __future__ import annotations

import torch

from tokamak_amd.kernels import ops


def linear(x: torch.Tensor, weight: torch.Tensor, out_dtype: torch.dtype | None = None,
           allow_partials: bool = False) -> torch.Tensor:
    """``x`` [M, K], ``weight`` [N, K] -> [M, N] in ``out_dtype`` (default: x's).

    With ``allow_partials`` the result may instead be float32 partial sums
    [P, M, N] that the consumer adds (the norm kernel and the q/k norm kernel do).
    """
    out_dtype = out_dtype or x.dtype
    m, n = x.shape[0], weight.shape[0]
    if m == 0:
        return torch.empty((0, n), dtype=out_dtype, device=x.device)
    if x.dtype == torch.float32:
        out = torch.empty((m, n), dtype=out_dtype, device=x.device)
        ops.gemm_tiled(x, weight, out)
        return out
    from tokamak_amd.kernels import gemm_bf16

    return gemm_bf16.gemm(x, weight, out_dtype, allow_partials)
