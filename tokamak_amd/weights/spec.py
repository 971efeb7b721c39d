"""What a part says about each tensor it wants from the checkpoint."""

from __future__ import annotations

from dataclasses import dataclass


@dataclass(frozen=True)
class TensorSpec:
    """``role`` says what kind of numbers the tensor holds, which fixes how the
    random-weights mode draws it: ``matrix`` (N(0, std)), ``vector`` (norm weights and
    the like: 1 + N(0, jitter)), ``table`` (integers).

    ``held`` says in which dtype the engine keeps it: ``"compute"`` (the engine's
    bfloat16 or float32), ``"float32"`` (whatever the checkpoint stores, so a tensor
    stored in 32-bit keeps its precision), ``"int32"``, or ``"stored"`` (as the checkpoint
    has it).  None takes the role's habit: matrices in the compute dtype, vectors in
    float32, tables as int32.  A matrix that must not be rounded (a router, a decay
    table) says ``held="float32"`` and stays a matrix.

    ``optional`` tensors may be absent; ``ignored`` ones may be present and are
    skipped (a tied head's own copy of the embedding)."""

    shape: tuple[int, ...]
    role: str = "matrix"
    optional: bool = False
    ignored: bool = False
    held: str | None = None

    def __post_init__(self) -> None:
        if self.role not in ("matrix", "vector", "table"):
            raise ValueError(f"role must be matrix, vector or table, got {self.role!r}")
        if self.held not in (None, "compute", "float32", "int32", "stored"):
            raise ValueError(f"held must be compute, float32, int32 or stored, got {self.held!r}")

    @property
    def holding(self) -> str:
        if self.held is not None:
            return self.held
        return {"matrix": "compute", "vector": "float32", "table": "int32"}[self.role]
