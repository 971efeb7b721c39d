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


def gated_linear(x: torch.Tensor, gate_up: torch.Tensor) -> torch.Tensor:
    """silu(x @ gate^T) * (x @ up^T) for ``gate_up`` = [gate; up] ([2I, K]) -> [M, I].

    bfloat16 with up to 64 rows: one fused weight-streaming kernel.  Otherwise
    the product, then the SiLU-gate kernel.
    """
    m = x.shape[0]
    inter = gate_up.shape[0] // 2
    out = torch.empty((m, inter), dtype=x.dtype, device=x.device)
    if m == 0:
        return out
    if x.dtype == torch.bfloat16 and m <= 64:
        from tokamak_amd.kernels import gemm_bf16

        if gemm_bf16.skinny_fits(x, gate_up):
            ops.gemm_stream_swiglu(x, gate_up, out)
            return out
    ops.silu_mul(linear(x, gate_up), out)
    return out
