"""bfloat16 matrix products with float32 accumulation."""

from __future__ import annotations

import torch

from tokamak_amd.kernels import ops

SKINNY_MAX_ROWS = 64
TARGET_WAVES = 4096   # waves wanted in flight for a weight-streaming product


def skinny_fits(x: torch.Tensor, weight: torch.Tensor) -> bool:
    k = x.shape[1]
    return (k % 8 == 0 and x.stride(0) % 8 == 0 and weight.stride(0) % 8 == 0
            and x.data_ptr() % 16 == 0 and weight.data_ptr() % 16 == 0)


def skinny_plan(m: int, n: int, k: int) -> tuple[int, int]:
    """(tiles of 16 weight rows per block, waves of a block that split K).

    More row tiles per block let the activation fragments be reused; more waves
    put more loads in flight when the matrix has few rows.  Chosen from
    measurements on the projection shapes of 0.6B to 32B models.
    """
    if m > 32:
        row_tiles = 4 if n >= 6144 else 2
    elif m <= 2 or n < 6144:
        row_tiles = 1
    else:
        row_tiles = 4 if n >= 65536 else 2
    blocks = -(-n // (16 * row_tiles))
    waves = 4
    while waves < 16 and blocks * waves < TARGET_WAVES:
        waves *= 2
    while waves > 1 and k // waves < 64:
        waves //= 2
    return row_tiles, waves


def gemm(x: torch.Tensor, weight: torch.Tensor, out: torch.Tensor) -> None:
    """out[M, N] = x[M, K] @ weight[N, K]^T; out is bfloat16 or float32.

    Up to 64 rows (decode batches, wanted logits rows): the hand-written
    weight-streaming MFMA kernel.  More rows with bfloat16 output: the library
    product torch binds (as the reference's nn.Linear does).  More rows with
    float32 output (many wanted logits rows): the skinny kernel, 64 rows at a time.
    """
    m = x.shape[0]
    n, k = weight.shape
    if skinny_fits(x, weight) and (m <= SKINNY_MAX_ROWS or out.dtype == torch.float32):
        row_tiles, waves = skinny_plan(min(m, SKINNY_MAX_ROWS), n, k)
        for at in range(0, m, SKINNY_MAX_ROWS):
            ops.gemm_skinny(x[at:at + SKINNY_MAX_ROWS], weight, out[at:at + SKINNY_MAX_ROWS],
                            row_tiles=row_tiles, waves=waves)
    elif out.dtype == torch.bfloat16:
        torch.matmul(x, weight.t(), out=out)
    else:
        ops.gemm_tiled(x, weight, out)
