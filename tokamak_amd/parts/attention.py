"""Grouped-query attention over a paged cache."""

from __future__ import annotations

import torch

from tokamak_amd.config.registry import register_part
from tokamak_amd.kernels import ops
from tokamak_amd.kernels.attention import (ATTENTION_WORK, check_page_size, decode_attention_fused, fused_decode_fits,
                                            paged_attention)
from tokamak_amd.kernels.linear import linear
from tokamak_amd.parts.base import CacheRequest, Fetch, Mixer, PositionData
from tokamak_amd.weights.spec import TensorSpec


class GQAAttention(Mixer):
    """q/k/v projections, optional per-head RMSNorm of q and k, rotation of q and k
    by the tables the layer's position encoding prepared (none: no rotation),
    causal softmax attention over the request's pages, o projection
    (reference: src/tokamak/model/transformer.py:22-86).

    Query head a reads kv head a // (num_heads / num_kv_heads).  Keys are cached
    after norm and rotation, values as projected (transformer.py:71-82).  The
    three projections are held as one [(nh + 2 nkv) hd, H] matrix.
    ``window``: None for full causal attention, W to see the last W positions.
    """

    capturable = True
    fuses_residual = True
    replayable = True

    def __init__(self, *, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 qk_norm_eps: float | None, softmax_scale: float, window: int | None,
                 dtype, device) -> None:
        super().__init__(dtype=dtype, device=device)
        if num_heads % num_kv_heads:
            raise ValueError(f"num_heads ({num_heads}) must be divisible by num_kv_heads ({num_kv_heads})")
        if head_dim % 16 or head_dim > 512:
            raise ValueError(f"head_dim must be a multiple of 16 and at most 512, got {head_dim}")
        self.hidden_size, self.num_heads, self.num_kv_heads = int(hidden_size), int(num_heads), int(num_kv_heads)
        self.head_dim = int(head_dim)
        self.qk_norm_eps = None if qk_norm_eps is None else float(qk_norm_eps)
        self.softmax_scale = float(softmax_scale)
        self.window = None if window is None else int(window)
        self.qkv: torch.Tensor | None = None
        self.o: torch.Tensor | None = None
        self.q_norm: torch.Tensor | None = None
        self.k_norm: torch.Tensor | None = None

    def expected_tensors(self, prefix: str) -> dict[str, TensorSpec]:
        h, nh, nkv, hd = self.hidden_size, self.num_heads, self.num_kv_heads, self.head_dim
        out = {
            prefix + "q_proj.weight": TensorSpec((nh * hd, h)),
            prefix + "k_proj.weight": TensorSpec((nkv * hd, h)),
            prefix + "v_proj.weight": TensorSpec((nkv * hd, h)),
            prefix + "o_proj.weight": TensorSpec((h, nh * hd)),
        }
        if self.qk_norm_eps is not None:
            out[prefix + "q_norm.weight"] = TensorSpec((hd,), role="vector")
            out[prefix + "k_norm.weight"] = TensorSpec((hd,), role="vector")
        return out

    def bind(self, prefix: str, fetch: Fetch) -> None:
        self.qkv = torch.cat([fetch(prefix + n + "_proj.weight") for n in "qkv"], dim=0).contiguous()
        self.o = fetch(prefix + "o_proj.weight")
        if self.qk_norm_eps is not None:
            self.q_norm = fetch(prefix + "q_norm.weight")
            self.k_norm = fetch(prefix + "k_norm.weight")

    def cache_request(self) -> CacheRequest:
        width = self.num_kv_heads * self.head_dim
        return CacheRequest.of(window=self.window, k=width, v=width)

    def step_planner(self):
        return ATTENTION_WORK

    def check_page_size(self, page_size: int) -> None:
        check_page_size(page_size)

    def pair_flops(self) -> float:
        # q.k and p.v: two multiply-adds per head and head element
        return 4.0 * self.num_heads * self.head_dim

    def forward(self, h, batch, store, writes_cache: bool = True,
                position: PositionData | None = None, add_into=None):
        nh, nkv, hd = self.num_heads, self.num_kv_heads, self.head_dim
        n = h.shape[0]
        weight = self.qkv if writes_cache else self.qkv[: nh * hd]
        qkv = linear(h, weight, allow_partials=True)
        cos = sin = None
        rotary_dim = 0
        if position is not None:
            if position.score_slopes is not None:
                raise ops.KernelError("this attention part has no kernel for a bias on the scores; "
                                      "it takes rotary tables or no position data")
            cos, sin, rotary_dim = position.cos, position.sin, position.rotary_dim
        tables = batch.block_tables[store.group]
        attended = torch.empty((n, nh * hd), dtype=h.dtype, device=h.device)
        if fused_decode_fits(h.dtype, hd, store.page_size, nh // nkv, self.window, rotary_dim, batch):
            # a step of decode tokens only: norm, rotation, cache write and attention in one kernel
            if decode_attention_fused(
                    qkv, self.q_norm, self.k_norm, cos, sin, store.arrays["k"], store.arrays["v"], tables, batch,
                    attended, num_heads=nh, num_kv_heads=nkv, head_dim=hd, rotary_dim=rotary_dim,
                    page_size=store.page_size, eps=self.qk_norm_eps or 0.0, scale=self.softmax_scale,
                    store=writes_cache):
                return linear(attended, self.o, allow_partials=True, add_into=add_into)
        q = torch.empty((n, nh * hd), dtype=h.dtype, device=h.device)
        ops.qknorm_rope_store(
            qkv, self.q_norm, self.k_norm, cos, sin, batch.positions, batch.req_of_token, tables, q,
            store.arrays["k"], store.arrays["v"], num_heads=nh, num_kv_heads=nkv, head_dim=hd,
            rotary_dim=rotary_dim, page_size=store.page_size,
            eps=self.qk_norm_eps or 0.0, store=writes_cache)
        paged_attention(q, store.arrays["k"], store.arrays["v"], tables, batch, attended,
                        num_heads=nh, num_kv_heads=nkv, head_dim=hd, page_size=store.page_size,
                        scale=self.softmax_scale, window=self.window)
        return linear(attended, self.o, allow_partials=True, add_into=add_into)


register_part("mixer", "gqa_attention", GQAAttention)
