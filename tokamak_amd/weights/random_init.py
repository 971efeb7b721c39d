"""Random-weights mode: write a model folder from a configuration and a seed."""

from __future__ import annotations

import json
from pathlib import Path
from typing import Any

import torch
from safetensors.torch import save_file

from tokamak_amd.config.registry import get_architecture
from tokamak_amd.weights.sources import RandomSource


def expected_tensors_of(plan) -> dict:
    """Tensor names and shapes of the model a plan describes (no device memory)."""
    from tokamak_amd.engine.model import LayeredModel

    return LayeredModel(plan, dtype=torch.float32, device="meta").expected_tensors()


def write_random_model(
    folder: str | Path,
    config: Any,
    seed: int,
    *,
    matrix_std: float = 0.02,
    vector_jitter: float = 0.0,
    dtype: torch.dtype = torch.bfloat16,
    eos_token_ids: tuple[int, ...] | None = None,
) -> Path:
    """Write ``config.json`` and ``model.safetensors`` for ``config`` (an
    architecture's typed config) with seeded random weights; return the folder.

    Matrices ~ N(0, matrix_std), norm weights 1 + N(0, vector_jitter), drawn in
    float32 and stored in ``dtype``.  A tied model gets no ``lm_head.weight``.
    """
    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    arch = get_architecture(config.architecture)
    if arch.to_json is None:
        raise ValueError(f"architecture {arch.name!r} cannot write a config.json")
    plan = arch.plan(config)
    expected = {n: s for n, s in expected_tensors_of(plan).items() if not s.ignored}
    source = RandomSource(expected, seed, matrix_std=matrix_std, vector_jitter=vector_jitter, dtype=dtype)
    tensors = {name: source.fetch(name).contiguous() for name in expected}
    save_file(tensors, str(folder / "model.safetensors"), metadata={"format": "pt"})
    (folder / "config.json").write_text(json.dumps(arch.to_json(config), indent=2) + "\n")
    eos = config.eos_token_ids if eos_token_ids is None else eos_token_ids
    if eos:
        (folder / "generation_config.json").write_text(json.dumps({"eos_token_id": list(eos)}) + "\n")
    return folder
