"""The benchmark's timed decoding runs the generation loop itself (``LLM.run``): on a tiny
model the steps it issues are those ``LLM.generate`` issues for the same requests, and the
tokens are the plain implementation's."""

import pytest

import plain_qwen3 as plain
from tiny import TINIES, make_folder

pytestmark = pytest.mark.gpu


def test_timed_decoding_is_the_generation_loop(tmp_path, monkeypatch):
    import bench
    from tokamak_amd import LLM, SamplingParams

    cfg = TINIES["B"]["config"]
    monkeypatch.setattr(bench, "PAGE_SIZE", 8)
    monkeypatch.setattr(bench, "PREFILL_TOKENS", 16)          # prompts of 40 tokens run in three portions
    batch, prompt_tokens, steps = 3, 40, 6
    built = bench.make_llm(cfg, "bfloat16", pool_tokens=256, max_requests=4, max_seq_len=64)
    assert built.runner.page_size == 8 and built.max_num_batched_tokens == 16 and built.max_seq_len == 64
    from tokamak_amd.kernels import ops
    assert ops._lt_tune == ops.LT_TUNE_CANDIDATES     # what the record calls tuned_products is on in this engine
    bench.make_llm(cfg, "bfloat16", pool_tokens=256, max_requests=4, max_seq_len=64, tune=False)
    assert ops._lt_tune == 1
    del built
    folder = make_folder(tmp_path, "B")       # weights the plain implementation can read
    llm = LLM(folder, dtype="float32", block_size=8, kv_pool_tokens=256, max_batch_size=4, max_seq_len=64,
              max_num_batched_tokens=16)
    made = []
    new_request = llm.new_request
    monkeypatch.setattr(llm, "new_request", lambda *a, **k: made.append(new_request(*a, **k)) or made[-1])

    logged = []
    step = llm.runner.step

    def logging_step(entries):
        logged.append([(e.request, len(e.tokens), e.feed, list(e.want)) for e in entries])
        return step(entries)

    monkeypatch.setattr(llm.runner, "step", logging_step)
    seconds = bench.decode_pass(llm, cfg.vocab_size, batch, prompt_tokens, steps, seed=3)
    assert seconds > 0
    timed_tokens = [list(r.generated) for r in made]
    timed = logged[-steps:]
    # every timed step is one token of every request; from the second on, still on the GPU
    assert timed[0] == [(r, 1, None, [0]) for r in range(batch)]
    assert all(s == [(r, 1, r, [0]) for r in range(batch)] for s in timed[1:])
    assert len(logged) == batch * 3 + steps
    llm.runner.manager.check()
    assert llm.runner.manager.num_free_pages() == llm.runner.manager.num_pages()

    # the same requests through generate(): the same decode steps, and the plain implementation's tokens
    prompts = [bench.random_prompt(cfg.vocab_size, prompt_tokens, 3 * 1000 + r) for r in range(batch)]
    logged.clear()
    outs = llm.generate(prompt_token_ids=prompts, use_tqdm=False,
                        sampling_params=SamplingParams(temperature=0.0, max_new_tokens=steps + 1, ignore_eos=True))
    # (there the requests start one after the other; the steps in which all three decode are the timed ones')
    decode_steps = [s for s in logged if len(s) == batch and all(n == 1 and fed is not None for _, n, fed, _ in s)]
    assert decode_steps and all(s == timed[1] for s in decode_steps)
    pcfg, w = plain.read_folder(folder)
    for out, prompt, tokens in zip(outs, prompts, timed_tokens):
        assert out.output_token_ids == tokens == plain.greedy(prompt, steps + 1, pcfg, w)
