"""A word-level tokenizer and a ChatML template written into a model folder, offline:
``tokenizer.json`` built with the ``tokenizers`` package, ``tokenizer_config.json`` with
``chat_template`` and ``eos_token``.  The folder then looks like a chat checkpoint's."""

from __future__ import annotations

import json
from pathlib import Path

WORDS = ("what does an inference engine do it runs tokens through layers and keeps keys values "
         "in pages user assistant hello world a b c").split()
SPECIALS = ["<unk>", "<|im_start|>", "<|im_end|>", "<think>", "</think>"]

# ChatML as chat checkpoints of this family write it: turns between <|im_start|> and
# <|im_end|>; with enable_thinking false an empty think block opens the answer
CHAT_TEMPLATE = (
    "{% for message in messages %}"
    "{{ '<|im_start|> ' + message['role'] + ' ' + message['content'] + ' <|im_end|> ' }}"
    "{% endfor %}"
    "{% if add_generation_prompt %}{{ '<|im_start|> assistant ' }}"
    "{% if enable_thinking is defined and enable_thinking is false %}{{ '<think> </think> ' }}{% endif %}"
    "{% endif %}"
)


def vocabulary() -> dict[str, int]:
    return {w: i for i, w in enumerate(SPECIALS + sorted(set(WORDS)))}


def add_tokenizer(folder: Path, *, template: bool = True, eos_token: str | None = "<|im_end|>") -> dict[str, int]:
    from tokenizers import Tokenizer, models, pre_tokenizers

    vocab = vocabulary()
    tok = Tokenizer(models.WordLevel(vocab, unk_token="<unk>"))
    tok.pre_tokenizer = pre_tokenizers.WhitespaceSplit()
    tok.add_special_tokens(SPECIALS)
    tok.save(str(Path(folder) / "tokenizer.json"))
    config = {}
    if template:
        config["chat_template"] = CHAT_TEMPLATE
    if eos_token is not None:
        config["eos_token"] = eos_token
    (Path(folder) / "tokenizer_config.json").write_text(json.dumps(config))
    return vocab
