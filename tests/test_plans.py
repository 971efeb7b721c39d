"""How products are cut into blocks (no GPU needed): the plan of splits and block sizes of
the weight-streaming product keeps its own rules at every size."""

import pytest

from tokamak_amd.kernels import ops
from tokamak_amd.kernels.gemm_bf16 import STREAM_TARGET_BLOCKS, stream_splits

SHAPES = [(4096, 1024), (1024, 2048), (1024, 3072), (6144, 2560), (2560, 9728), (6144, 4096), (4096, 4096),
          (4096, 12288), (10240, 5120), (5120, 8192), (5120, 25600), (151936, 4096), (151936, 1024), (48, 264), (130, 8)]


@pytest.mark.parametrize("n,k", SHAPES)
@pytest.mark.parametrize("m", [1, 8, 16, 17, 32, 33, 48, 64])
def test_splits_stay_within_the_chunks_and_fill_the_gpu_evenly(n, k, m):
    chunks = -(-k // 256)
    waves = ops.stream_waves(m, k, False, n)
    assert waves in (4, 8)
    splits = stream_splits(n, k, m)
    assert 1 <= splits <= max(1, chunks)
    blocks = -(-n // (16 * waves))
    if m > 16 and 2 * n * k >= ops.STREAM_SMALL_MATRIX_BYTES:
        # what runs at once: two blocks of four waves a CU (an eighth over is taken), one of eight
        limit = STREAM_TARGET_BLOCKS * 9 // 8 if waves == 4 else STREAM_TARGET_BLOCKS // 2
        assert splits == 1 or splits * blocks <= limit
        assert splits == 1 or chunks // splits >= 2
        assert waves == (8 if m > 32 and n <= 256 * 128 else 4)
    else:
        assert waves == 4


def test_the_gated_product_takes_eight_waves_only_when_it_has_the_columns():
    assert ops.stream_waves(64, 4096, True, 12288) == 8
    assert ops.stream_waves(64, 1024, True, 3072) == 4      # too few columns for blocks of eight
    assert ops.stream_waves(32, 4096, True, 12288) == 4
    assert ops.stream_waves(8, 4096, True, 12288) == 4
