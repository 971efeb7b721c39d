"""Registries: architecture name -> model description, part name -> part class.

The reference recognises architectures by membership in a frozenset and
switches on the name inside one model class (reference:
src/tokamak/config.py:20-26,92-96,124).  Here an architecture is an entry that
parses its own ``config.json`` keys and returns a ``ModelPlan``; parts are
looked up by the names the plan uses.
"""

from __future__ import annotations

import json
from dataclasses import dataclass, field
from pathlib import Path
from typing import Any, Callable, Mapping

from tokamak_amd.config.model_config import ModelPlan


@dataclass(frozen=True)
class Architecture:
    """``parse`` turns (config.json dict, eos ids) into the typed config;
    ``plan`` turns that typed config into a ``ModelPlan``; ``to_json`` writes
    the typed config back as a ``config.json`` dict (used by the random-weights
    folder writer).  ``presets``: named typed configs (shapes for the
    random-weights mode of the command line and the benchmark).  ``chat_prompt``:
    user text -> prompt text, used when a model folder has no chat template."""

    name: str
    parse: Callable[[dict[str, Any], tuple[int, ...]], Any]
    plan: Callable[[Any], ModelPlan]
    to_json: Callable[[Any], dict[str, Any]] | None = None
    presets: Mapping[str, Any] = field(default_factory=dict)
    chat_prompt: Callable[[str], str] | None = None


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


def preset_names() -> list[str]:
    """Names of every registered architecture's presets."""
    _ensure_builtin()
    return sorted(n for a in _ARCHITECTURES.values() for n in a.presets)


def find_preset(name: str) -> tuple[Architecture, Any]:
    """(architecture, typed config) of the preset ``name``, whichever architecture has it."""
    _ensure_builtin()
    for arch in _ARCHITECTURES.values():
        if name in arch.presets:
            return arch, arch.presets[name]
    raise ValueError(f"unknown preset {name!r}; presets: {', '.join(preset_names())}")


def _as_ids(raw) -> tuple[int, ...]:
    if isinstance(raw, bool) or raw is None:
        return ()
    if isinstance(raw, int):
        return (raw,)
    if isinstance(raw, list):
        return tuple(int(x) for x in raw if isinstance(x, int) and not isinstance(x, bool))
    return ()


def _read_json(path: Path) -> dict:
    if not path.is_file():
        return {}
    raw = json.loads(path.read_text())
    return raw if isinstance(raw, dict) else {}


def _tokenizer_eos(folder: Path) -> tuple[int, ...]:
    """The id of ``tokenizer_config.json``'s ``eos_token`` in ``tokenizer.json``."""
    token = _read_json(folder / "tokenizer_config.json").get("eos_token")
    if isinstance(token, dict):
        token = token.get("content")
    if not isinstance(token, str):
        return ()
    tok = _read_json(folder / "tokenizer.json")
    for added in tok.get("added_tokens") or []:
        if isinstance(added, dict) and added.get("content") == token and isinstance(added.get("id"), int):
            return (added["id"],)
    vocab = (tok.get("model") or {}).get("vocab")
    if isinstance(vocab, dict) and isinstance(vocab.get(token), int):
        return (vocab[token],)
    return ()


def read_eos_token_ids(folder: Path) -> tuple[int, ...]:
    """EOS ids of a model folder: ``generation_config.json``'s ``eos_token_id`` (an
    int or a list); else ``config.json``'s; else the tokenizer's EOS token; else
    none, and requests then stop on length only.

    Reference: src/tokamak/engine/llm.py:244-263 (generation config first, then
    the tokenizer's ``eos_token_id``).
    """
    folder = Path(folder)
    for ids in (_as_ids(_read_json(folder / "generation_config.json").get("eos_token_id")),
                _as_ids(_read_json(folder / "config.json").get("eos_token_id")),
                _tokenizer_eos(folder)):
        if ids:
            return ids
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
