"""The text path on the GPU: ``generate(prompts=...)``, the tokenizer's EOS, ``output_text``,
and the command line's ``--prompt`` through the chat template
(reference: examples/basic_generation.py:25-42, src/tokamak/engine/llm.py:244-263,501-536)."""

import pytest

import plain_qwen3 as plain
from text_util import add_tokenizer
from tiny import make_folder

pytestmark = pytest.mark.gpu
pytest.importorskip("tokenizers")
pytest.importorskip("jinja2")


@pytest.fixture(scope="module")
def chat_folder(tmp_path_factory):
    folder = make_folder(tmp_path_factory.mktemp("text"), "A")
    vocab = add_tokenizer(folder)
    return folder, vocab


def test_generate_from_text_tokenizes_decodes_and_stops_on_the_tokenizers_eos(chat_folder):
    from tokamak_amd import LLM, SamplingParams

    folder, vocab = chat_folder
    cfg, w = plain.read_folder(folder)
    llm = LLM(folder, dtype="float32", max_seq_len=96)
    assert llm.tokenizer is not None
    assert llm.eos_token_ids == (vocab["<|im_end|>"],)      # no generation_config.json: the tokenizer's
    texts = ["what does an inference engine do", "it runs tokens through layers"]
    outs = llm.generate(texts, SamplingParams(temperature=0.0, max_new_tokens=10, ignore_eos=True), use_tqdm=False)
    words = {i: word for word, i in vocab.items()}
    for out, text in zip(outs, texts):
        ids = [vocab[word] for word in text.split()]
        assert out.prompt == text and out.prompt_token_ids == ids
        assert out.output_token_ids == plain.greedy(ids, 10, cfg, w)
        # the text is the output ids decoded, special tokens dropped (ids beyond the
        # tokenizer's vocabulary, which a random model may draw, decode to nothing)
        expect = " ".join(words[t] for t in out.output_token_ids if t in words and not words[t].startswith("<"))
        assert out.output_text == expect

    # a single string is one prompt; with the EOS id made the greedy run's third token, the
    # request stops there and keeps it
    free_run = plain.greedy([vocab["hello"], vocab["world"]], 8, cfg, w)
    llm.eos_token_ids = (free_run[2],)
    out = llm.generate("hello world", SamplingParams(temperature=0.0, max_new_tokens=8), use_tqdm=False)
    assert len(out) == 1
    stop = free_run.index(free_run[2])
    assert out[0].output_token_ids == free_run[:stop + 1] and out[0].finish_reason.value == "stop"


def test_prompts_need_a_tokenizer(tmp_path):
    from tokamak_amd import LLM

    llm = LLM(make_folder(tmp_path, "A"), dtype="float32")
    assert llm.tokenizer is None
    with pytest.raises(ValueError, match="tokenizer.json"):
        llm.generate("hello")
    with pytest.raises(ValueError, match="exactly one"):
        llm.generate("hello", prompt_token_ids=[[1]])


def test_command_line_prompt_goes_through_the_chat_template(chat_folder, capsys):
    from tokamak_amd import LLM, SamplingParams, cli

    folder, vocab = chat_folder
    rc = cli.main(["--model", str(folder), "--prompt", "hello world", "--temperature", "0",
                   "--max-new-tokens", "6", "--dtype", "float32", "--quiet"])
    printed = capsys.readouterr().out
    assert rc == 0
    assert "[prompt]\nhello world\n" in printed and "[completion (" in printed

    # what it printed is the completion of the templated prompt
    llm = LLM(folder, dtype="float32")
    prompt = llm.chat_prompt("hello world")
    assert prompt == "<|im_start|> user hello world <|im_end|> <|im_start|> assistant <think> </think> "
    out = llm.generate(prompt, SamplingParams(temperature=0.0, max_new_tokens=6), use_tqdm=False)[0]
    assert out.prompt_token_ids == [vocab[t] for t in prompt.split()]
    completion = printed.split("]\n")[-1].rstrip("\n")
    assert completion == (out.output_text or "")


def test_progress_bar_counts_finished_requests(chat_folder):
    from tokamak_amd import LLM, SamplingParams

    folder, _ = chat_folder
    llm = LLM(folder, dtype="float32")
    llm.generate(["a b c", "hello world", "it runs"], SamplingParams(temperature=0.0, max_new_tokens=3))
    assert llm.last_progress == "3/3"           # the bar is on by default, as the reference's
