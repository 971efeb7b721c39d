"""Bind checkpoint tensors to a model by name, with full-coverage validation.

Reference: src/tokamak/model/loader.py:54-95 raises on the first unexpected,
mismatched or missing tensor.  Here one ``WeightError`` lists all three kinds
at once, before any tensor is read.
"""

from __future__ import annotations

from typing import Callable, Mapping

import torch

from tokamak_amd.weights.spec import TensorSpec


class WeightError(ValueError):
    """Checkpoint and model disagree; ``missing``, ``unexpected`` and
    ``mismatched`` hold the tensor names of each kind."""

    def __init__(self, missing, unexpected, mismatched) -> None:
        self.missing = sorted(missing)
        self.unexpected = sorted(unexpected)
        self.mismatched = sorted(mismatched)
        lines = ["checkpoint does not match the model:"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): {self.missing}")
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): {self.unexpected}")
        for name, got, want in self.mismatched:
            lines.append(f"  wrong shape for {name!r}: checkpoint {tuple(got)} vs model {tuple(want)}")
        super().__init__("\n".join(lines))


def validate(expected: Mapping[str, TensorSpec], found: Mapping[str, tuple]) -> None:
    """Raise ``WeightError`` unless ``found`` covers ``expected`` exactly."""
    missing = [n for n, s in expected.items() if n not in found and not (s.optional or s.ignored)]
    unexpected = [n for n in found if n not in expected]
    mismatched = [
        (n, found[n][0], s.shape)
        for n, s in expected.items()
        if n in found and not s.ignored and tuple(found[n][0]) != tuple(s.shape)
    ]
    if missing or unexpected or mismatched:
        raise WeightError(missing, unexpected, mismatched)


def target_dtype(spec: TensorSpec, stored: torch.dtype, compute_dtype: torch.dtype) -> torch.dtype:
    return {"int32": torch.int32, "float32": torch.float32, "stored": stored, "compute": compute_dtype}[spec.holding]


def load_weights(model, source, *, dtype: torch.dtype, device: str | torch.device) -> int:
    """Validate ``source`` against ``model.expected_tensors()`` and bind.

    ``model.bind(fetch)`` asks for each tensor by checkpoint name; ``fetch``
    returns it on ``device`` in the dtype its role prescribes.  Returns the
    number of tensors read.
    """
    expected = model.expected_tensors()
    found = source.names()
    validate(expected, found)
    count = 0

    def fetch(name: str) -> torch.Tensor | None:
        nonlocal count
        spec = expected[name]
        if name not in found:
            return None
        count += 1
        tensor = source.fetch(name)
        return tensor.to(device=device, dtype=target_dtype(spec, tensor.dtype, dtype)).contiguous()

    model.bind(fetch)
    return count


Fetch = Callable[[str], "torch.Tensor | None"]
