"""Dispatch of paged attention to the kernel that fits the shape."""

from __future__ import annotations

import torch

from tokamak_amd.kernels import ops

MFMA_HEAD_DIMS = (64, 128)
SPLIT_KEYS = 256          # fewest keys a split of a decode token's context holds
TARGET_DECODE_WAVES = 4096  # waves wanted in flight; beyond that splits only cost a merge


def mfma_fits(dtype, head_dim, page_size, group, window) -> bool:
    return (dtype == torch.bfloat16 and head_dim in MFMA_HEAD_DIMS and page_size >= 16
            and page_size & (page_size - 1) == 0 and group <= 16 and window is None)


def decode_split(num_decode: int, num_kv_heads: int, max_len: int) -> tuple[int, int]:
    """(keys per split, number of splits) for the decode tokens of a step: as few
    splits as fill the GPU (one wave per request, kv head and split), never
    shorter than SPLIT_KEYS."""
    most = max(1, -(-max_len // SPLIT_KEYS))
    nsplit = min(most, max(1, -(-TARGET_DECODE_WAVES // (num_decode * num_kv_heads))))
    split = -(-max_len // nsplit)
    split = -(-split // 16) * 16
    return split, max(1, -(-max_len // split))


def paged_attention(q, k_cache, v_cache, block_tables, batch, out, *, num_heads, num_kv_heads,
                    head_dim, page_size, scale, window=None) -> None:
    """out[n] = softmax(q[n] . K[0..pos_n] * scale) V, per head, over the pages
    of each token's request.

    bfloat16 with head size 64 or 128: the MFMA kernel, once over the single
    (decode) tokens with their context split, once over 16-token tiles of the
    prompt portions.  Everything else: the generic float32-arithmetic kernel.
    """
    if mfma_fits(q.dtype, head_dim, page_size, num_heads // num_kv_heads, window):
        common = dict(num_heads=num_heads, num_kv_heads=num_kv_heads, head_dim=head_dim,
                      page_size=page_size, scale=scale)
        if batch.num_decode:
            split, nsplit = decode_split(batch.num_decode, num_kv_heads, batch.max_decode_len)
            ops.attention_mfma("heads", q, k_cache, v_cache, block_tables, batch.positions,
                               batch.req_of_token, batch.decode_tokens, None, batch.num_decode, out,
                               split_keys=split, num_splits=nsplit, **common)
        if batch.num_tiles:
            ops.attention_mfma("tokens", q, k_cache, v_cache, block_tables, batch.positions,
                               batch.req_of_token, batch.tile_first, batch.tile_count, batch.num_tiles,
                               out, split_keys=1 << 30, num_splits=1, **common)
        return
    ops.paged_attention_generic(
        q, k_cache, v_cache, block_tables, batch.positions, batch.req_of_token, out,
        num_heads=num_heads, num_kv_heads=num_kv_heads, head_dim=head_dim, page_size=page_size,
        scale=scale, window=window)
