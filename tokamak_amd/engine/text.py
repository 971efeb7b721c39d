"""Text in and out of a model folder: its tokenizer and its chat template.

The reference leaves both to a library tokenizer object (src/tokamak/engine/llm.py:150-152
loads it; examples/basic_generation.py:25-30 asks it for the chat prompt).  Here the
folder's ``tokenizer.json`` is read with the ``tokenizers`` package and the template
string of ``tokenizer_config.json`` is rendered in a sandbox; nothing of the folder is
executed.
"""

from __future__ import annotations

import json
from pathlib import Path


def load_tokenizer(folder: Path | None):
    """The folder's ``tokenizer.json`` as a ``tokenizers.Tokenizer``; None if the folder
    has none (or the package is absent): callers then take token ids only."""
    if folder is None:
        return None
    path = Path(folder) / "tokenizer.json"
    if not path.is_file():
        return None
    try:
        from tokenizers import Tokenizer
    except ImportError:
        return None
    return Tokenizer.from_file(str(path))


def folder_chat_template(folder: Path | None) -> str | None:
    if folder is None:
        return None
    path = Path(folder) / "tokenizer_config.json"
    if not path.is_file():
        return None
    raw = json.loads(path.read_text())
    template = raw.get("chat_template") if isinstance(raw, dict) else None
    return template if isinstance(template, str) else None


def chat_prompt(folder: Path | None, architecture, user_text: str) -> str:
    """``user_text`` as a single user turn, ready to tokenize.  The folder's own chat
    template when it has one, rendered with ``add_generation_prompt=True`` and
    ``enable_thinking=False`` as the reference's example asks
    (examples/basic_generation.py:25-30); else the architecture's; else the text as it is."""
    template = folder_chat_template(folder)
    if template is not None:
        from jinja2.sandbox import ImmutableSandboxedEnvironment

        env = ImmutableSandboxedEnvironment(trim_blocks=True, lstrip_blocks=True)
        return env.from_string(template).render(
            messages=[{"role": "user", "content": user_text}], add_generation_prompt=True,
            enable_thinking=False)
    if architecture is not None and architecture.chat_prompt is not None:
        return architecture.chat_prompt(user_text)
    return user_text
