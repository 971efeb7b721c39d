"""Token embedding and the output head."""

from __future__ import annotations

import torch

from tokamak_amd.config.registry import register_part
from tokamak_amd.kernels import ops
from tokamak_amd.kernels.linear import linear
from tokamak_amd.parts.base import Embedding, Fetch, Head
from tokamak_amd.weights.spec import TensorSpec


class TokenEmbedding(Embedding):
    """Plain row gather into the float32 residual stream, no scaling
    (reference: src/tokamak/model/transformer.py:140)."""

    capturable = True

    def __init__(self, *, vocab_size: int, dim: int, dtype, device) -> None:
        super().__init__(dtype=dtype, device=device)
        self.vocab_size, self.dim = int(vocab_size), int(dim)
        self.weight: torch.Tensor | None = None

    def expected_tensors(self, prefix: str) -> dict[str, TensorSpec]:
        return {prefix + "weight": TensorSpec((self.vocab_size, self.dim))}

    def bind(self, prefix: str, fetch: Fetch) -> None:
        self.weight = fetch(prefix + "weight")

    def tied_matrix(self) -> torch.Tensor:
        return self.weight

    def forward(self, batch) -> torch.Tensor:
        resid = torch.empty((batch.num_tokens, self.dim), dtype=torch.float32, device=self.device)
        ops.embed_gather(self.weight, batch.token_ids, resid)
        return resid


class LinearHead(Head):
    """logits = h @ W^T in float32; a tied head uses the embedding matrix itself
    (reference: src/tokamak/model/transformer.py:154-156,173-176)."""

    capturable = True

    def __init__(self, *, vocab_size: int, dim: int, tied: bool, dtype, device) -> None:
        super().__init__(dtype=dtype, device=device)
        self.vocab_size, self.dim, self.tied = int(vocab_size), int(dim), bool(tied)
        self.weight: torch.Tensor | None = None

    def expected_tensors(self, prefix: str) -> dict[str, TensorSpec]:
        # a tied checkpoint may still carry its own copy: it is skipped
        # (reference: src/tokamak/model/loader.py:79-80)
        return {prefix + "weight": TensorSpec((self.vocab_size, self.dim), ignored=self.tied)}

    def bind(self, prefix: str, fetch: Fetch) -> None:
        if not self.tied:
            self.weight = fetch(prefix + "weight")

    def tie(self, embedding: Embedding) -> None:
        weight = embedding.tied_matrix()
        if tuple(weight.shape) != (self.vocab_size, self.dim):
            raise ValueError(f"a tied head of {(self.vocab_size, self.dim)} cannot share an embedding "
                             f"matrix of {tuple(weight.shape)}")
        self.weight = weight

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        return linear(h, self.weight, out_dtype=torch.float32)


register_part("embedding", "token_embedding", TokenEmbedding)
register_part("head", "linear_head", LinearHead)
