"""Options of the entry point that are checked before anything touches the GPU
(names and defaults: reference src/tokamak/engine/llm.py:106-122)."""

import pytest

from tokamak_amd import LLM


@pytest.mark.parametrize("option, value", [
    ("kv_backend", "contiguous"), ("scheduling", "static"), ("attention_backend", "triton"),
    ("attention_policy", "sliding_window"), ("draft_model", "some/model"),
])
def test_the_references_other_choices_are_refused_by_name(tmp_path, option, value):
    with pytest.raises(ValueError, match=option):
        LLM(tmp_path, **{option: value})


def test_cpu_is_refused(tmp_path):
    with pytest.raises(ValueError, match="GPU only"):
        LLM(tmp_path, device="cpu")


def test_missing_folder_is_an_error_and_nothing_is_downloaded(tmp_path):
    with pytest.raises(FileNotFoundError, match="no download"):
        LLM(tmp_path / "Qwen" / "Qwen3-0.6B")


def test_sizes_are_checked(tmp_path):
    with pytest.raises(ValueError, match="block_size"):
        LLM(tmp_path, block_size=0)
    with pytest.raises(ValueError, match="max_batch_size"):
        LLM(tmp_path, max_batch_size=0)
