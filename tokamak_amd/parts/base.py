"""Interfaces of the parts a layer is made of.

A part is built from its ``PartSpec`` parameters plus the engine's dtype and
device; it names the checkpoint tensors it wants (``expected_tensors``), takes
them (``bind``) and computes (``forward``).  No part knows which model it is
in: sizes and constants arrive as parameters, checkpoint names arrive as a
prefix, and everything about the running batch arrives in the ``StepBatch``.

* ``Embedding.forward(batch)``: the float32 residual stream [N, H] of the step's
  tokens (token rows; an absolute position encoding would be added here, from
  ``batch.positions``).
* ``Norm.forward(resid, delta, ...)``: adds ``delta`` into the float32 residual
  stream and returns the normed activations in the compute dtype.  ``delta`` is
  a sub-layer's output: [N, H] in the compute dtype or float32, or float32
  partial sums [P, N, H] of a split-K product, which the norm adds.
* ``PositionEncoding.prepare(batch)``: per-step ``PositionData`` (rotary tables,
  per-head score slopes), computed once per step and shared by every layer whose
  encoding has the same parameters.  The block hands it to its mixer.
* ``Mixer.forward(h, batch, store, writes_cache, position)``: token mixing.  It
  may own paged cache (``cache_request``) and/or fixed-size per-request state
  (``state_request``); it sees its own storage only.
* ``FeedForward.forward(h, batch)``: token-wise map [N, H] -> [N, H].
* ``Block.forward(resid, pending, ...)``: the arrangement of a layer's parts,
  which it receives as a dict by role.

A part whose kernels want the step cut into work of their own shape (tiles of a
portion's tokens, chunks of a scan) declares a ``StepPlanner``; what page sizes its
kernels take it says in ``check_page_size``.  The engine asks; it knows neither.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable

import torch

from tokamak_amd.engine.batch import StepPlanner  # noqa: F401  (part of the parts' interface)
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
    # ``replayable``: besides, the part launches all its work through ``kernels.ops`` (no
    # routine of torch's computes for it) and decides nothing from what differs between two
    # layers with equal parameters, so the launches of one layer, with another layer's
    # tensors put in, are that layer's (engine/layer_replay.py).
    replayable = False
    # Whether the part takes part in the fusion of the residual add and the norm into the
    # products around them (kernels/linear.py).  A norm that says so takes ``Added`` as its
    # ``delta`` (the sum is already in the stream) and a keyword ``defer`` (it may then
    # return a ``DeferredNorm`` instead of a tensor), and offers ``sink(resid)``.  A mixer or
    # feed-forward that says so takes a ``DeferredNorm`` as its input ``h`` (it hands it to
    # ``linear`` / ``gated_linear`` only, before the stream is written again) and a keyword
    # ``add_into``: a ``StreamSink`` for its last product, whose ``Added`` it returns.  A
    # block that says so takes ``Added`` as ``pending``, a keyword ``then`` (the norm that
    # reads the stream after the block, or None) and names its first norm ``entry_norm``.
    # Parts that do not say so never meet these types.
    fuses_residual = False

    def __init__(self, *, dtype: torch.dtype, device: torch.device | str) -> None:
        self.dtype = dtype
        self.device = torch.device(device)

    def expected_tensors(self, prefix: str) -> dict[str, TensorSpec]:
        return {}

    def bind(self, prefix: str, fetch: Fetch) -> None:
        pass

    def step_planner(self) -> StepPlanner | None:
        """The planner of the work lists this part's kernels read, or None."""
        return None

    def check_page_size(self, page_size: int) -> None:
        """Raise ``ValueError`` if the part's kernels cannot work with cache pages of
        ``page_size`` tokens."""


@dataclass(frozen=True)
class PagedArray:
    """One paged array of a mixer: elements per token, and its dtype (None: the
    engine's compute dtype)."""

    elems_per_token: int
    dtype: torch.dtype | None = None


@dataclass(frozen=True)
class CacheRequest:
    """What a mixer asks of the paged cache for one cache slot.

    ``arrays``: (name, PagedArray) pairs; the arrays of one request may differ in
    width and dtype (keys and values of unlike sizes, a compressed latent beside
    its rotary part).  The mixer reads ``store.arrays[name]``, laid out
    [num_pages, elems_per_token * page_size].  ``window``: None to keep every
    token, W if only the last W positions are ever read."""

    arrays: tuple[tuple[str, PagedArray], ...]
    window: int | None = None

    @classmethod
    def of(cls, window: int | None = None, **arrays: int | PagedArray) -> CacheRequest:
        return cls(tuple((n, a if isinstance(a, PagedArray) else PagedArray(int(a))) for n, a in arrays.items()),
                   window)

    def bytes_per_token(self, default_dtype: torch.dtype) -> int:
        return sum(a.elems_per_token * torch.empty((), dtype=a.dtype or default_dtype).element_size()
                   for _, a in self.arrays)


@dataclass(frozen=True)
class StateArray:
    """One array of a mixer's fixed-size per-request state."""

    shape: tuple[int, ...]
    dtype: torch.dtype = torch.float32


@dataclass
class PositionData:
    """What a position encoding hands to a mixer for one step.

    ``cos``/``sin``: float32 [N, rotary_dim / 2] tables for a mixer that rotates
    queries and keys (half-split pairing), or None.  ``score_slopes``: float32
    [heads] for a mixer that adds ``slope * (key position - query position)`` to its
    scores, or None.  A mixer refuses what it has no kernel for."""

    cos: torch.Tensor | None = None
    sin: torch.Tensor | None = None
    rotary_dim: int = 0
    score_slopes: torch.Tensor | None = None
    extra: dict = field(default_factory=dict)


class Embedding(Part):
    def forward(self, batch) -> torch.Tensor:
        raise NotImplementedError

    def tied_matrix(self) -> torch.Tensor:
        """The [vocab, dim] matrix a head shares with this embedding when the two are tied."""
        raise NotImplementedError(f"{type(self).__name__} has no matrix to tie a head to")


class Head(Part):
    def forward(self, h: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError

    def tie(self, embedding: Embedding) -> None:
        raise NotImplementedError


class Norm(Part):
    def forward(self, resid: torch.Tensor, delta: torch.Tensor | None, *,
                rows: torch.Tensor | None = None, write_resid: bool = True) -> torch.Tensor:
        raise NotImplementedError


class PositionEncoding(Part):
    def prepare(self, batch) -> PositionData:
        raise NotImplementedError


class Mixer(Part):
    def cache_request(self) -> CacheRequest | None:
        """Paged storage per token, or None."""
        return None

    def state_request(self) -> dict[str, StateArray] | None:
        """Arrays of the fixed-size per-request state by name, or None.  The mixer
        reads ``store.state[name][batch.state_slots[r]]``; every array is zero when
        a request is admitted."""
        return None

    def pair_flops(self) -> float:
        """Floating-point operations per (query token, visible earlier token) pair of one
        call, for the measurement's count of a step's work; 0 for a mixer whose work does
        not grow with the context."""
        return 0.0

    def forward(self, h: torch.Tensor, batch, store, writes_cache: bool = True,
                position: PositionData | None = None) -> torch.Tensor:
        raise NotImplementedError


class FeedForward(Part):
    def forward(self, h: torch.Tensor, batch) -> torch.Tensor:
        raise NotImplementedError


class Block:
    """Arrangement of one layer's parts.

    ``roles``: names of the parts it needs; ``optional``: of those it can do
    without.  ``parts`` holds the built parts by role.  ``mixers`` holds those that are
    mixers, by role, in the order the plan names them: a layer call brings one cache slot
    for each.  With one mixer (or none) ``forward`` receives that slot's ``SlotStore`` as
    ``store`` and ``mixer`` names it; with several, ``store`` is a dict of ``SlotStore`` by
    the mixers' roles.
    """

    roles: tuple[str, ...] = ()
    optional: tuple[str, ...] = ()
    fuses_residual = False      # see Part.fuses_residual
    replays_parts = False       # the block's own forward is replayable, see Part.replayable
    entry_norm: "Norm | None" = None   # the norm that reads the stream first, if the block fuses

    def __init__(self, parts: dict[str, Part]) -> None:
        missing = [r for r in self.roles if r not in parts]
        unknown = [r for r in parts if r not in self.roles and r not in self.optional]
        if missing or unknown:
            raise ValueError(f"{type(self).__name__} needs parts {sorted(self.roles)} "
                             f"(optional: {sorted(self.optional)}); missing {missing}, unknown {unknown}")
        self.parts = dict(parts)
        self.mixers: dict[str, Mixer] = {role: p for role, p in parts.items() if isinstance(p, Mixer)}
        self.mixer: Mixer | None = next(iter(self.mixers.values())) if len(self.mixers) == 1 else None
        # a block's launches are replayed only if the block itself says so and all its parts do
        self.replayable = bool(type(self).replays_parts) and all(p.replayable for p in parts.values())

    def forward(self, resid: torch.Tensor, pending: torch.Tensor | None, batch, store,
                writes_cache: bool) -> torch.Tensor | None:
        """Run the layer on the residual stream ``resid`` (float32, updated in
        place by the norms); ``pending`` is the previous layer's last sub-layer
        output, not yet added.  Returns this layer's last sub-layer output, to be
        added by whoever norms next."""
        raise NotImplementedError
