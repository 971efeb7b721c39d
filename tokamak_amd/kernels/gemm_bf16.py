"""bfloat16 matrix products with float32 accumulation."""

from __future__ import annotations

import torch

from tokamak_amd.kernels import ops

SKINNY_MAX_ROWS = 64
TARGET_WAVES = 4096     # waves wanted in flight for the direct-operand kernel
STREAM_MIN_ROWS_OUT = 1024    # weight rows from which the LDS-staged kernel (64 rows a block) is used
STREAM_TARGET_BLOCKS = 512


def skinny_fits(x: torch.Tensor, weight: torch.Tensor) -> bool:
    k = x.shape[1]
    return (k % 8 == 0 and x.stride(0) % 8 == 0 and weight.stride(0) % 8 == 0
            and x.data_ptr() % 16 == 0 and weight.data_ptr() % 16 == 0)


def skinny_plan(m: int, n: int, k: int) -> tuple[int, int]:
    """(tiles of 16 weight rows per block, waves of a block that split K) for the
    direct-operand kernel.  More row tiles per block let the activation fragments
    be reused; more waves put more loads in flight when the matrix has few rows.
    Chosen from measurements on the projection shapes of 0.6B to 32B models."""
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


def _fill(total: int) -> float:
    """How well `total` blocks of four waves use the GPU: two a CU run at full rate, so up to 512
    count by their number; beyond, the CUs that get one block more than the others set the time, so
    a count just under the next multiple of 256 is good and one just over it is the worst (80 row
    blocks of a 14B-shaped down projection: 480 blocks 29 us, 560 blocks 35 us, 720 blocks 32 us);
    every further block a CU costs a little by itself (partial sums, shorter shares)."""
    room = max(STREAM_TARGET_BLOCKS, -(-total // 256) * 256)
    return total / room * 0.95 ** ((room - STREAM_TARGET_BLOCKS) // 256)


def stream_splits(n: int, k: int, m: int = 1) -> int:
    """Shares of K for the LDS-staged kernel so that enough blocks exist, and no more.

    Up to 32 rows (blocks of four waves): of the numbers of shares that K's chunks of 256 allow, the
    one whose blocks fill the CUs most evenly (``_fill``): 512 blocks or a little less, else a
    little less than 768.  17 to 32 rows of a large matrix: never fewer than two chunks a share,
    since every split also writes (and the next kernel reads) float32 partial sums of all rows.
    Small matrices (the projections of a 0.6B-shaped model) at any number of rows likewise, down
    to one chunk a share: such a product is read in one memory round trip then, and its time is
    round trips, not bytes.  More rows: a block holds more LDS and one block of six or eight waves
    runs on a CU, so a few blocks beyond the 256 CUs cost a whole further round (measured at
    32B-shaped sizes with 64 rows: 280 blocks of eight waves take 80 us where 240 take 57): at most
    256 blocks, never fewer than two chunks a share.  Against the best of every split measured on
    the projection shapes of 1.7B to 32B models at 4 to 32 rows this is within 1 % on average and
    10 % at worst (a small matrix with 32 rows)."""
    chunks = -(-k // 256)
    blocks = -(-n // (16 * ops.stream_waves(m, k, False, n)))
    small = 2 * n * k < ops.STREAM_SMALL_MATRIX_BYTES
    if m <= 32 or (small and m <= SKINNY_MAX_ROWS):
        if blocks >= STREAM_TARGET_BLOCKS:
            return 1
        least_share = 1 if m <= 16 or small else min(2, chunks)
        best, best_fill = 1, _fill(blocks)
        for share in range(chunks, least_share - 1, -1):        # chunks a share, fewest splits first
            splits = -(-chunks // share)
            if splits > 64:
                break
            fill = _fill(blocks * splits)
            if fill > best_fill:
                best, best_fill = splits, fill
        return best
    splits = max(1, STREAM_TARGET_BLOCKS // 2 // blocks)
    return max(1, min(splits, chunks // 2))


STREAM_PARTIALS_ROWS = 96           # rows up to which the split streaming product beats the library at every size
STREAM_PARTIALS_BIG = 64 << 20      # ... and the bytes of a matrix from which it does up to 128 rows


def stream_pays_beyond_64_rows(m: int, n: int, k: int) -> bool:
    """Whether a product of 65 to 128 rows whose reader adds partial sums goes to the streaming
    kernel (five to eight tiles of 16 rows, eight waves a block) rather than to the library.
    Against the library's fastest candidate, q/k/v, o and down of 1.7B- to 32B-shaped layers are
    10 to 40 % faster at 65 to 96 rows; at 128 rows the large matrices still are (down of a
    32B-shaped layer 82 against 119 us) and the small ones are level or behind, and the partial
    sums cost their reader a few microseconds more.  Whole decode steps: batch 80 at 1.7B / 8B /
    14B / 32B widths +1 / +4 / +13 / +7 %, batch 128 -4 / -3 / +4 / +5 % if every product
    took this path, hence the limit on small matrices."""
    if not SKINNY_MAX_ROWS < m <= ops.STREAM_MAX_ROWS or n < STREAM_MIN_ROWS_OUT:
        return False
    return m <= STREAM_PARTIALS_ROWS or 2 * n * k >= STREAM_PARTIALS_BIG


def gemm(x: torch.Tensor, weight: torch.Tensor, out_dtype: torch.dtype, allow_partials: bool = False) -> torch.Tensor:
    """x[M, K] @ weight[N, K]^T -> [M, N] in ``out_dtype``; or, if the caller can
    add them (``allow_partials``), float32 partial sums [P, M, N] of a split-K product.

    Up to 64 rows (decode batches, wanted logits rows): hand-written
    weight-streaming MFMA kernels: the LDS-staged one, split over K into partial
    sums when the matrix has few rows and the caller adds them; the
    direct-operand one for very small matrices.  65 to 128 rows, if the caller adds partial
    sums: the same kernel with five to eight tiles of 16 rows where it was measured to pay
    (``stream_pays_beyond_64_rows``).  Else more than 64 rows
    with bfloat16 output: the library product (hipBLASLt, as the reference's
    nn.Linear ends in a library; csrc/blas_lt.hip); with float32 output: 128 rows at a time.
    """
    m = x.shape[0]
    n, k = weight.shape
    dev = x.device
    fits = skinny_fits(x, weight)
    if fits and allow_partials and (m <= SKINNY_MAX_ROWS or stream_pays_beyond_64_rows(m, n, k)):
        splits = stream_splits(n, k, m)
        if splits > 1:
            out = torch.empty((splits, m, n), dtype=torch.float32, device=dev)
            used = ops.gemm_stream(x, weight, out, splits=splits)
            return out[:used]
    if fits and (m <= SKINNY_MAX_ROWS or out_dtype == torch.float32):
        out = torch.empty((m, n), dtype=out_dtype, device=dev)
        # (a logits head over 65 to 128 rows at once: 320-365 us at 8B width, 490-530 in two passes)
        step = ops.STREAM_MAX_ROWS if n >= STREAM_MIN_ROWS_OUT else SKINNY_MAX_ROWS
        for at in range(0, m, step):
            xs, os_ = x[at:at + step], out[at:at + step]
            if n >= STREAM_MIN_ROWS_OUT:
                ops.gemm_stream(xs, weight, os_)
            else:
                row_tiles, waves = skinny_plan(xs.shape[0], n, k)
                ops.gemm_skinny(xs, weight, os_, row_tiles=row_tiles, waves=waves)
        return out
    out = torch.empty((m, n), dtype=out_dtype, device=dev)
    if out_dtype == torch.bfloat16:
        # hipBLASLt with kept plans and measured algorithms; shapes it has nothing for
        # (rows that are not 16-byte aligned, say) go through torch's binding of it
        if not (skinny_fits(x, weight) and ops.gemm_library(x, weight, out)):
            ops.not_replayable()
            torch.matmul(x, weight.t(), out=out)
    else:
        ops.gemm_tiled(x, weight, out)
    return out
