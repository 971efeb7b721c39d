"""Interfaces of the parts a layer is made of.

A part is built from its ``PartSpec`` parameters plus the engine's dtype and
device; it names the checkpoint tensors it wants (``expected_tensors``), takes
them (``bind``) and computes (``forward``).  No part knows which model it is
in: sizes and constants arrive as parameters, checkpoint names arrive as a
prefix, and everything about the running batch arrives in the ``StepBatch``.

* ``Norm.forward(resid, delta, ...)``: adds ``delta`` into the float32 residual
  stream and returns the normed activations in the compute dtype.  ``delta`` is
  a sub-layer's output: [N, H] in the compute dtype or float32, or float32
  partial sums [P, N, H] of a split-K product, which the norm adds.
* ``Mixer.forward(h, batch, store, writes_cache)``: token mixing.  It may own
  paged cache (``cache_request``) and/or fixed-size per-request state
  (``state_shape``); it sees its own storage only.
* ``FeedForward.forward(h, batch)``: token-wise map [N, H] -> [N, H].
* ``PositionEncoding.prepare(batch)``: per-step data (e.g. rotary tables),
  computed once per step and shared by every layer that uses the same encoding.
* ``Block.forward(resid, pending, ...)``: the arrangement of the above.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Callable

import torch

from tokamak_amd.weights.spec import TensorSpec

Fetch = Callable[[str], "torch.Tensor | None"]


class Part:
    """Common base: parameters, expected tensors, binding.

    ``capturable``: the part's ``forward`` only launches work on the current
    stream (no host synchronisation, no data-dependent host decisions), so a
    decode step through it may be recorded into a HIP graph.  A model is captured
    only if every part of it says so.
    """

    capturable = False

    def __init__(self, *, dtype: torch.dtype, device: torch.device | str) -> None:
        self.dtype = dtype
        self.device = torch.device(device)

    def expected_tensors(self, prefix: str) -> dict[str, TensorSpec]:
        return {}

    def bind(self, prefix: str, fetch: Fetch) -> None:
        pass


@dataclass(frozen=True)
class CacheRequest:
    """What a mixer asks of the paged cache for one cache slot.

    ``arrays``: name -> elements per page as a function of the page size is
    fixed by the mixer: ``page_elems(page_size)`` per array.  ``window``: None to
    keep every token, W if only the last W positions are ever read."""

    arrays: tuple[str, ...]
    elems_per_token: int
    window: int | None = None


class Norm(Part):
    def forward(self, resid: torch.Tensor, delta: torch.Tensor | None, *,
                rows: torch.Tensor | None = None, write_resid: bool = True) -> torch.Tensor:
        raise NotImplementedError


class PositionEncoding(Part):
    def prepare(self, batch) -> object:
        raise NotImplementedError


class Mixer(Part):
    def cache_request(self) -> CacheRequest | None:
        """Paged storage per token, or None."""
        return None

    def state_shape(self) -> tuple[int, ...] | None:
        """Shape of the fixed-size per-request state, or None."""
        return None

    def forward(self, h: torch.Tensor, batch, store, writes_cache: bool = True) -> torch.Tensor:
        raise NotImplementedError


class FeedForward(Part):
    def forward(self, h: torch.Tensor, batch) -> torch.Tensor:
        raise NotImplementedError


class Block:
    """Arrangement of one layer's parts."""

    def __init__(self, mixer: Mixer, feed_forward: FeedForward, mixer_norm: Norm,
                 feed_forward_norm: Norm) -> None:
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.mixer_norm = mixer_norm
        self.feed_forward_norm = feed_forward_norm

    def forward(self, resid: torch.Tensor, pending: torch.Tensor | None, batch, store,
                writes_cache: bool) -> torch.Tensor:
        raise NotImplementedError
