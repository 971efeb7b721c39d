"""Dispatch of paged attention to the kernel that fits the shape."""

from __future__ import annotations

import torch

from tokamak_amd.kernels import ops


def paged_attention(q, k_cache, v_cache, block_tables, batch, out, *, num_heads, num_kv_heads,
                    head_dim, page_size, scale, window=None) -> None:
    """out[n] = softmax(q[n] . K[0..pos_n] * scale) V, per head, over the pages
    of each token's request."""
    ops.paged_attention_generic(
        q, k_cache, v_cache, block_tables, batch.positions, batch.req_of_token, out,
        num_heads=num_heads, num_kv_heads=num_kv_heads, head_dim=head_dim, page_size=page_size,
        scale=scale, window=window)
