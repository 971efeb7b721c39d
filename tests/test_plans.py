"""How products are cut into blocks (no GPU needed): the plan of splits and block sizes of
the weight-streaming product keeps its own rules at every size."""

import pytest

from tokamak_amd.kernels import ops
from tokamak_amd.kernels.gemm_bf16 import STREAM_TARGET_BLOCKS, _fill, stream_splits

SHAPES = [(4096, 1024), (1024, 2048), (1024, 3072), (6144, 2560), (2560, 9728), (6144, 4096), (4096, 4096),
          (4096, 12288), (10240, 5120), (5120, 8192), (5120, 25600), (151936, 4096), (151936, 1024), (48, 264), (130, 8)]


@pytest.mark.parametrize("n,k", SHAPES)
@pytest.mark.parametrize("m", [1, 8, 16, 17, 32, 33, 48, 64])
def test_splits_stay_within_the_chunks_and_fill_the_gpu_evenly(n, k, m):
    chunks = -(-k // 256)
    waves = ops.stream_waves(m, k, False, n)
    assert waves in (4, 6, 8)
    splits = stream_splits(n, k, m)
    assert 1 <= splits <= max(1, chunks)
    blocks = -(-n // (16 * waves))
    large = 2 * n * k >= ops.STREAM_SMALL_MATRIX_BYTES
    if m > 32 and large:
        # one block of six or eight waves a CU
        assert splits == 1 or splits * blocks <= STREAM_TARGET_BLOCKS // 2
        assert splits == 1 or chunks // splits >= 2
        if n <= 256 * 128:
            # six waves only where one round of them covers a tenth more of the CUs than one of eight
            six, eight = ops.stream_fill(n, k, 6)[0], ops.stream_fill(n, k, 8)[0]
            assert waves == (6 if six >= 1.1 * eight else 8)
        else:
            assert waves == 4
        return
    assert waves == 4
    used = -(-chunks // -(-chunks // splits))       # the kernel's shares: none is empty
    assert used == splits                           # the plan names the number that runs
    if m > 16 and large and splits > 1:
        assert -(-chunks // splits) >= 2
    # no other number of shares fills the CUs more evenly
    least = 1 if m <= 16 or not large else 2
    if blocks < STREAM_TARGET_BLOCKS:
        for share in range(least, chunks + 1):
            other = -(-chunks // share)
            assert other > 64 or _fill(blocks * other) <= _fill(blocks * splits)


def test_splits_of_the_measured_shapes():
    # (output columns, K, rows) -> shares of K that were the fastest, or within a few percent of it
    cases = {
        (6144, 4096, 8): 8, (4096, 4096, 8): 8, (4096, 12288, 8): 8, (6144, 4096, 24): 8, (4096, 12288, 32): 8,     # 8B
        (7168, 5120, 8): 4, (5120, 5120, 8): 5, (5120, 17408, 8): 6, (5120, 17408, 32): 6,                          # 14B
        (10240, 5120, 16): 3, (5120, 8192, 4): 6, (5120, 25600, 16): 6,                                             # 32B
        (6144, 2560, 16): 5, (2560, 4096, 4): 16, (2560, 4096, 24): 8, (2560, 9728, 16): 19,                        # 4B
        (2048, 6144, 4): 24, (2048, 6144, 32): 12,                                                                  # 1.7B
        (151936, 4096, 8): 1,                                                                                       # a head
    }
    for (n, k, m), splits in cases.items():
        assert stream_splits(n, k, m) == splits, (n, k, m)


def test_the_gated_product_picks_its_block_size_by_rows_columns_and_row_length():
    # (rows, K, output columns) -> waves: the shapes the rule was measured on
    cases = {
        (1, 1024, 3072): 2, (16, 1024, 3072): 2, (48, 1024, 3072): 2, (64, 1024, 3072): 2,       # 0.6B
        (8, 2048, 6144): 2, (32, 2048, 6144): 2, (48, 2048, 6144): 2, (64, 2048, 6144): 4,        # 1.7B
        (8, 2560, 9728): 2, (32, 2560, 9728): 2, (48, 2560, 9728): 6,                             # 4B
        (1, 4096, 12288): 4, (16, 4096, 12288): 4, (32, 4096, 12288): 4, (64, 4096, 12288): 6,    # 8B: rows of 8 KB; 256 blocks of six
        (8, 5120, 17408): 2, (24, 5120, 17408): 4, (64, 5120, 17408): 6,                          # 14B
        (8, 5120, 25600): 2, (32, 5120, 25600): 4, (33, 5120, 25600): 8,                          # 32B
    }
    for (rows, k, n), waves in cases.items():
        assert ops.stream_waves(rows, k, True, n) == waves, (rows, k, n)


def test_six_waves_where_they_fill_the_gpu_better():
    # q/k/v of an 8B-shaped layer: 64 row blocks of six waves x 4 shares of K = 256 blocks, of eight 48 x 4
    assert ops.stream_fill(6144, 4096, 6) == (1.0, 4) and ops.stream_fill(6144, 4096, 8) == (0.75, 4)
    assert ops.stream_waves(64, 4096, False, 6144) == 6 and stream_splits(6144, 4096, 64) == 4
    # o and down of the same layer are 256 blocks of eight already
    assert ops.stream_waves(64, 4096, False, 4096) == 8 and ops.stream_waves(64, 12288, False, 4096) == 8
    # the gated product at 32B: three rounds of six lose to two of eight
    assert ops.stream_waves(64, 5120, True, 25600) == 8


def test_the_group_form_of_prefill_attention_is_taken_where_it_was_measured_to_pay():
    from tokamak_amd.kernels.attention import group_form_pays

    wide = lambda tokens: -(-tokens // 32)
    # (query heads a kv head, kv heads, tokens of the portion, longest context) -> group form
    cases = {
        (4, 8, 2048, 2048): True, (4, 8, 2048, 32768): True, (4, 8, 256, 1280): True, (4, 8, 128, 5000): False,   # 8B, 4B
        (4, 8, 2048, 1000): False,                                                                               # short walks
        (5, 8, 2048, 2048): True, (5, 8, 512, 1536): True, (5, 8, 256, 4352): False, (5, 8, 128, 16512): False,   # 14B: too few blocks
        (8, 8, 2048, 2048): True, (8, 8, 1024, 1024): False, (8, 8, 1024, 2048): True, (8, 8, 512, 1536): False,  # 32B
        (8, 8, 512, 4608): True, (8, 8, 256, 16640): False,
        (2, 8, 512, 4608): True, (2, 8, 1024, 17408): True, (2, 8, 1024, 1024): False, (2, 8, 2048, 6144): False,  # 0.6B, 1.7B
        (3, 1, 2048, 2048): True, (16, 2, 2048, 2048): True,
    }
    for (group, nkv, tokens, longest), want in cases.items():
        assert group_form_pays(group, nkv, wide(tokens), longest) == want, (group, nkv, tokens, longest)


def test_decode_splits_follow_how_the_blocks_fill_the_rounds():
    from tokamak_amd.kernels.attention import DECODE_WAVES, decode_split

    for requests in (1, 2, 7, 8, 16, 17, 31, 32, 33, 40, 64):
        for kv_heads in (1, 2, 8):
            for longest in (1, 255, 256, 257, 600, 2049, 2560, 8192, 40960):
                split, nsplit = decode_split(requests, kv_heads, longest)
                assert split % (16 * DECODE_WAVES) == 0 and nsplit >= 1 and split * nsplit >= longest
                assert split * (nsplit - 1) < longest            # no split past the longest request
    # 32 requests x 8 kv heads are one block a CU: no split; one request more is 264 blocks, whose
    # last eight would take as long again: split, so that the last round is short
    assert decode_split(32, 8, 2560)[1] == 1 and decode_split(64, 8, 2560)[1] == 1
    assert decode_split(33, 8, 2560)[1] >= 3
    # few requests: as many splits as fill the GPU, fewer when each split is only a few tiles long
    assert decode_split(8, 8, 2560)[1] == 4 and decode_split(1, 8, 2560)[1] >= 8
    assert decode_split(8, 8, 300)[1] <= 2
    assert decode_split(1, 2, 32768)[1] >= 32


def test_the_keys_of_few_tiles_are_split_over_blocks():
    from tokamak_amd.kernels.attention import tile_split

    none = (1 << 30, 1)
    # (tiles of 16 tokens, blocks of the narrow form a tile, longest context)
    assert tile_split(4, 2, 40960) == (512, 80)             # four tiles: pieces of 512 keys
    assert tile_split(16, 16, 16640)[1] == 8                # 256 tokens, 64 query heads: eight pieces
    assert tile_split(8, 40, 16512)[1] == 7                 # 128 tokens, five heads a kv head
    assert tile_split(16, 16, 1280) == none                 # pieces would be shorter than 1,024 keys
    assert tile_split(8, 8, 1100)[1] == 2                   # few blocks: pieces of 512 and more
    assert tile_split(64, 16, 16384) == none                # 1,024 blocks fill the GPU unsplit
    for tiles, per_tile, longest in ((4, 2, 40960), (16, 16, 16640), (35, 8, 5037), (3, 1, 1024)):
        split, nsplit = tile_split(tiles, per_tile, longest)
        if nsplit > 1:
            assert split % 64 == 0 and (nsplit - 1) * split < longest <= nsplit * split


def test_the_streaming_product_takes_65_to_128_rows_where_it_was_measured_to_pay():
    from tokamak_amd.kernels.gemm_bf16 import stream_pays_beyond_64_rows as pays

    # up to 96 rows at every width; to 128 for matrices of 64 MB and more; never the tiny ones
    for n, k in ((4096, 1024), (2048, 6144), (6144, 4096), (5120, 25600)):
        assert not pays(64, n, k) and pays(65, n, k) and pays(96, n, k) and not pays(129, n, k)
    assert not pays(97, 6144, 4096) and not pays(128, 4096, 4096)            # q/k/v and o of 8B: 50 and 34 MB
    assert pays(128, 4096, 12288) and pays(97, 7168, 5120) and pays(128, 5120, 25600)
    assert not pays(80, 48, 4096)                                            # fewer output columns than a block
    # the plan of such a product: blocks of eight waves, one a CU, at least two chunks a share
    for n, k, m in ((6144, 4096, 80), (4096, 12288, 128), (5120, 25600, 96), (2048, 6144, 70)):
        assert ops.stream_waves(m, k, False, n) == 8
        splits = stream_splits(n, k, m)
        assert splits > 1 and splits * -(-n // 128) <= 256 and -(-k // 256) // splits >= 2
