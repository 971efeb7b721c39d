"""The text side of a model folder without a GPU: tokenizer, chat template, EOS from the
tokenizer (reference: examples/basic_generation.py:25-30, src/tokamak/engine/llm.py:244-263)."""

import json

import pytest

from text_util import add_tokenizer
from tiny import make_folder

pytest.importorskip("tokenizers")
pytest.importorskip("jinja2")


@pytest.fixture()
def folder(tmp_path):
    return make_folder(tmp_path, "A")


def test_tokenizer_is_read_from_the_folder(folder):
    from tokamak_amd.engine import text

    assert text.load_tokenizer(folder) is None          # no tokenizer.json yet
    vocab = add_tokenizer(folder)
    tok = text.load_tokenizer(folder)
    ids = tok.encode("what does an inference engine do").ids
    assert ids == [vocab[w] for w in "what does an inference engine do".split()]
    assert tok.decode(ids, skip_special_tokens=True) == "what does an inference engine do"
    # special tokens are single ids, and decoding drops them
    ids = tok.encode("<|im_start|> user hello <|im_end|>").ids
    assert ids == [vocab["<|im_start|>"], vocab["user"], vocab["hello"], vocab["<|im_end|>"]]
    assert tok.decode(ids, skip_special_tokens=True) == "user hello"


def test_chat_prompt_renders_the_folders_template_without_thinking(folder):
    from tokamak_amd.config import get_architecture
    from tokamak_amd.engine import text

    arch = get_architecture("Qwen3ForCausalLM")
    add_tokenizer(folder)
    got = text.chat_prompt(folder, arch, "hello world")
    assert got == "<|im_start|> user hello world <|im_end|> <|im_start|> assistant <think> </think> "


def test_chat_prompt_falls_back_to_the_architectures(folder):
    from tokamak_amd.config import get_architecture
    from tokamak_amd.engine import text

    arch = get_architecture("Qwen3ForCausalLM")
    add_tokenizer(folder, template=False)
    got = text.chat_prompt(folder, arch, "hello world")
    assert got == arch.chat_prompt("hello world")
    assert got.startswith("<|im_start|>user\nhello world<|im_end|>\n<|im_start|>assistant\n")
    assert "<think>\n\n</think>" in got                  # thinking off, as the reference's example asks
    assert text.chat_prompt(None, None, "as it is") == "as it is"


def test_a_template_cannot_reach_outside_its_sandbox(folder):
    from jinja2.exceptions import SecurityError

    from tokamak_amd.engine import text

    add_tokenizer(folder)
    (folder / "tokenizer_config.json").write_text(json.dumps(
        {"chat_template": "{{ messages.__class__.__mro__ }}"}))
    with pytest.raises(SecurityError):
        text.chat_prompt(folder, None, "x")


def test_eos_comes_from_generation_config_then_config_then_tokenizer(folder):
    from tokamak_amd.config.registry import load_model_description, read_eos_token_ids

    assert read_eos_token_ids(folder) == ()
    vocab = add_tokenizer(folder)
    assert read_eos_token_ids(folder) == (vocab["<|im_end|>"],)
    _, cfg, plan = load_model_description(folder)
    assert cfg.eos_token_ids == plan.eos_token_ids == (vocab["<|im_end|>"],)
    raw = json.loads((folder / "config.json").read_text())
    raw["eos_token_id"] = 7
    (folder / "config.json").write_text(json.dumps(raw))
    assert read_eos_token_ids(folder) == (7,)
    (folder / "generation_config.json").write_text(json.dumps({"eos_token_id": [11, 12]}))
    assert read_eos_token_ids(folder) == (11, 12)
