"""What a part says about each tensor it wants from the checkpoint."""

from __future__ import annotations

from dataclasses import dataclass


@dataclass(frozen=True)
class TensorSpec:
    """``role``: ``matrix`` (held in the engine's compute dtype), ``vector``
    (norm weights and the like: held in float32 whatever the checkpoint stores,
    so a tensor stored in 32-bit keeps its precision), ``table`` (integers,
    held as int32).  ``optional`` tensors may be absent; ``ignored`` ones may be
    present and are skipped (a tied head's own copy of the embedding)."""

    shape: tuple[int, ...]
    role: str = "matrix"
    optional: bool = False
    ignored: bool = False
