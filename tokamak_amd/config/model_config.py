"""Typed model descriptions.

Two layers of description live here:

* ``ModelPlan`` is what the engine runs: which parts make each layer (by role:
  mixer, feed-forward, norms, position encoding ...) and which block arranges
  them, in which order layers are called and which cache slot each call uses.  It is pure data; nothing in it names an
  architecture.
* An architecture's own frozen config dataclass (``Qwen3Config`` in
  ``tokamak_amd.models.qwen3``) is parsed from the keys of its ``config.json``
  and turned into a plan by the architecture entry in the registry.

The reference keeps one flat ``ModelConfig`` for three architectures
(reference: src/tokamak/config.py:29-126); here every number a part needs is a
parameter of that part's ``PartSpec``.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any


def _freeze(value: Any) -> Any:
    if isinstance(value, dict):
        return tuple(sorted((k, _freeze(v)) for k, v in value.items()))
    if isinstance(value, (list, tuple)):
        return tuple(_freeze(v) for v in value)
    return value


@dataclass(frozen=True)
class PartSpec:
    """Name of a registered part plus its constructor parameters."""

    kind: str
    params: tuple[tuple[str, Any], ...] = ()

    @classmethod
    def of(cls, kind: str, **params: Any) -> PartSpec:
        return cls(kind, tuple(sorted((k, _freeze(v)) for k, v in params.items())))

    def as_dict(self) -> dict[str, Any]:
        return dict(self.params)

    def __getitem__(self, key: str) -> Any:
        for k, v in self.params:
            if k == key:
                return v
        raise KeyError(key)


@dataclass(frozen=True)
class SubPart:
    """One part of a layer: the registry family it is looked up in, its
    ``PartSpec``, and the sub-prefix of its checkpoint tensors inside the
    layer's own prefix.  ``shared``: every sub-part of the model with the same
    family and spec is one object (for parts without tensors whose per-step work,
    like a position encoding's tables, should be done once for all layers)."""

    family: str
    spec: PartSpec
    prefix: str = ""
    shared: bool = False


@dataclass(frozen=True)
class LayerSpec:
    """One layer: parts by role, and the block that arranges them.

    ``parts`` maps a role name to a ``SubPart``; which roles exist is between the
    architecture's plan and the block it names (``block.kind``): the pre-norm block
    asks for ``mixer_norm``, ``mixer``, ``feed_forward_norm``, ``feed_forward`` and
    takes an optional ``position``; a block with four norms, with one norm feeding
    two branches, or with no feed-forward simply names other roles.  Nothing else
    in the engine knows the role names.
    """

    parts: tuple[tuple[str, SubPart], ...]
    block: PartSpec = field(default_factory=lambda: PartSpec.of("pre_norm"))

    @classmethod
    def of(cls, block: PartSpec | None = None, **roles: SubPart) -> LayerSpec:
        return cls(tuple(roles.items()), block if block is not None else PartSpec.of("pre_norm"))

    def role(self, name: str) -> SubPart:
        for role, part in self.parts:
            if role == name:
                return part
        raise KeyError(name)


@dataclass(frozen=True)
class LayerCall:
    """One entry of the run order.

    ``layer`` indexes ``ModelPlan.layers`` (the weights); the same layer may be
    called more than once.  ``cache`` is the cache slot the call's mixer uses;
    two calls with the same slot share what is stored there.  A layer whose block
    holds several mixers brings a tuple of slots, one for each mixer in the order
    the layer names them.  A call with ``writes_cache=False`` only reads its slots
    (it attends over keys and values another call stored) and stores nothing itself.
    """

    layer: int
    cache: int | tuple[int, ...]
    writes_cache: bool = True

    @property
    def slots(self) -> tuple[int, ...]:
        return self.cache if isinstance(self.cache, tuple) else (self.cache,)


@dataclass(frozen=True)
class ModelPlan:
    """Everything the engine needs to build and run a model."""

    vocab_size: int
    hidden_size: int
    max_position_embeddings: int
    tie_word_embeddings: bool
    embedding: PartSpec
    layers: tuple[LayerSpec, ...]
    order: tuple[LayerCall, ...]
    final_norm: PartSpec
    head: PartSpec
    # checkpoint names; ``layer_prefix`` is formatted with the layer index
    embedding_prefix: str
    layer_prefix: str
    final_norm_prefix: str
    head_prefix: str
    eos_token_ids: tuple[int, ...] = ()

    def __post_init__(self) -> None:
        for call in self.order:
            if not 0 <= call.layer < len(self.layers):
                raise ValueError(f"run order names layer {call.layer}, model has {len(self.layers)}")
        written = {slot for call in self.order if call.writes_cache for slot in call.slots}
        for call in self.order:
            for slot in call.slots:
                if not call.writes_cache and slot not in written:
                    raise ValueError(f"cache slot {slot} is read but never written")

    @property
    def num_cache_slots(self) -> int:
        return 1 + max((slot for c in self.order for slot in c.slots), default=-1)


def default_order(num_layers: int) -> tuple[LayerCall, ...]:
    """Each layer once, in index order, each with a cache slot of its own."""
    return tuple(LayerCall(i, i) for i in range(num_layers))
