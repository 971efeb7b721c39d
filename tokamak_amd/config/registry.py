"""Registries: architecture name -> model description, part name -> part class.

The reference recognises architectures by membership in a frozenset and
switches on the name inside one model class (reference:
src/tokamak/config.py:20-26,92-96,124).  Here an architecture is an entry that
parses its own ``config.json`` keys and returns a ``ModelPlan``; parts are
looked up by the names the plan uses.
"""

from __future__ import annotations

import json
from dataclasses import dataclass
from pathlib import Path
from typing import Any, Callable

from tokamak_amd.config.model_config import ModelPlan


@dataclass(frozen=True)
class Architecture:
    """``parse`` turns (config.json dict, eos ids) into the typed config;
    ``plan`` turns that typed config into a ``ModelPlan``; ``to_json`` writes
    the typed config back as a ``config.json`` dict (used by the random-weights
    folder writer)."""

    name: str
    parse: Callable[[dict[str, Any], tuple[int, ...]], Any]
    plan: Callable[[Any], ModelPlan]
    to_json: Callable[[Any], dict[str, Any]] | None = None


_ARCHITECTURES: dict[str, Architecture] = {}
_PARTS: dict[tuple[str, str], type] = {}

PART_FAMILIES = ("mixer", "feed_forward", "norm", "position", "block", "embedding", "head")


def register_architecture(arch: Architecture, *, replace: bool = False) -> None:
    if arch.name in _ARCHITECTURES and not replace:
        raise ValueError(f"architecture {arch.name!r} is already registered")
    _ARCHITECTURES[arch.name] = arch


def get_architecture(name: str) -> Architecture:
    _ensure_builtin()
    try:
        return _ARCHITECTURES[name]
    except KeyError:
        supported = ", ".join(sorted(_ARCHITECTURES))
        raise ValueError(f"Unsupported architecture {name!r}; supported: {supported}") from None


def supported_architectures() -> list[str]:
    _ensure_builtin()
    return sorted(_ARCHITECTURES)


def register_part(family: str, kind: str, cls: type, *, replace: bool = False) -> None:
    if family not in PART_FAMILIES:
        raise ValueError(f"unknown part family {family!r}; families: {PART_FAMILIES}")
    if (family, kind) in _PARTS and not replace:
        raise ValueError(f"{family} part {kind!r} is already registered")
    _PARTS[(family, kind)] = cls


def get_part(family: str, kind: str) -> type:
    _ensure_builtin()
    try:
        return _PARTS[(family, kind)]
    except KeyError:
        known = sorted(k for f, k in _PARTS if f == family)
        raise ValueError(f"unknown {family} part {kind!r}; registered: {known}") from None


_builtin_loaded = False


def _ensure_builtin() -> None:
    global _builtin_loaded
    if _builtin_loaded:
        return
    _builtin_loaded = True
    import tokamak_amd.models  # noqa: F401  (registers architectures)
    import tokamak_amd.parts  # noqa: F401  (registers parts)


def read_eos_token_ids(folder: Path) -> tuple[int, ...]:
    """EOS ids from ``generation_config.json`` (an int or a list), else none.

    Reference: src/tokamak/engine/llm.py:244-263 (the tokenizer fallback is not
    reproduced: token ids are this engine's contract, a tokenizer is optional).
    """
    path = Path(folder) / "generation_config.json"
    if not path.is_file():
        return ()
    raw = json.loads(path.read_text()).get("eos_token_id")
    if isinstance(raw, bool):
        return ()
    if isinstance(raw, int):
        return (raw,)
    if isinstance(raw, list):
        return tuple(int(x) for x in raw)
    return ()


def load_model_description(folder: str | Path) -> tuple[Architecture, Any, ModelPlan]:
    """Read ``config.json`` in ``folder``; return (architecture, typed config, plan)."""
    folder = Path(folder)
    path = folder / "config.json"
    if not path.is_file():
        raise FileNotFoundError(f"no config.json under {folder}")
    raw = json.loads(path.read_text())
    names = raw.get("architectures") or []
    name = names[0] if names else "<missing>"
    arch = get_architecture(name)
    config = arch.parse(raw, read_eos_token_ids(folder))
    return arch, config, arch.plan(config)
