"""Generation through the entry point: greedy equals the plain implementation,
lengths and stop rules, seeded sampling, preemption is invisible."""

import pytest
import torch

import plain_qwen3 as plain
from replay_util import random_ids
from tiny import TINIES, make_folder

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("gen")
    return {k: make_folder(root, k) for k in TINIES}


@pytest.mark.parametrize("which, lengths, new", [("A", [5, 17, 33], 8), ("B", [1, 9, 40, 70], 12)])
def test_greedy_generation_matches_plain(folders, which, lengths, new):
    from tokamak_amd import LLM, SamplingParams

    folder = folders[which]
    cfg, w = plain.read_folder(folder)
    prompts = [random_ids(cfg["vocab_size"], n, 40 + i) for i, n in enumerate(lengths)]
    llm = LLM(folder, dtype="float32", block_size=TINIES[which]["page_size"], kv_pool_tokens=512,
              max_batch_size=4, max_num_batched_tokens=32, prefill_chunk=16)
    outs = llm.generate(prompt_token_ids=prompts,
                        sampling_params=SamplingParams(temperature=0.0, max_new_tokens=new, ignore_eos=True))
    assert [o.request_id for o in outs] == list(range(len(prompts)))
    for o, p in zip(outs, prompts):
        assert o.prompt_token_ids == p
        assert o.output_token_ids == plain.greedy(p, new, cfg, w)
        assert o.finish_reason.value == "length" and len(o.output_token_ids) == new
        assert o.ttft_s is not None and o.latency_s >= o.ttft_s
    llm.runner.manager.check()
    assert llm.runner.manager.num_free_pages() == llm.runner.manager.num_pages()


def test_bfloat16_greedy_picks_a_token_within_rounding_of_the_best(folders):
    """Every greedily generated bfloat16 token, checked against the plain float32 logits
    of the sequence so far: it is the best token, or one whose logit lies within twice
    the replay tests' bfloat16 bound (2e-3 + 2 % of the row's scale) of the best.  With
    a vocabulary of 331 and logits spread over the row's scale, a systematic error picks
    tokens far below that."""
    from tokamak_amd import LLM, SamplingParams
    from replay_util import TOL

    folder = folders["C"]
    cfg, w = plain.read_folder(folder)
    prompts = [random_ids(cfg["vocab_size"], n, 70 + i) for i, n in enumerate([12, 50])]
    llm = LLM(folder, dtype="bfloat16", kv_pool_tokens=1024)
    outs = llm.generate(prompt_token_ids=prompts, sampling_params=SamplingParams(temperature=0.0, max_new_tokens=6, ignore_eos=True))
    bound = TOL["bfloat16"]
    exact = 0
    for o, p in zip(outs, prompts):
        assert len(o.output_token_ids) == 6
        for i, token in enumerate(o.output_token_ids):
            row = plain.logits(p + o.output_token_ids[:i], cfg, w)[-1]
            slack = 2 * (bound["tol_abs"] + bound["tol_rel_to_scale"] * float(row.abs().max()))
            assert float(row[token]) >= float(row.max()) - slack, f"token {i} of a {len(p)}-token prompt"
            exact += int(token == int(row.argmax()))
    assert exact >= 9          # near-ties aside, the tokens are the plain implementation's


def test_stop_rules(folders, tmp_path):
    from tokamak_amd import LLM, SamplingParams
    import json, shutil

    folder = tmp_path / "with_eos"
    shutil.copytree(folders["A"], folder)
    cfg, w = plain.read_folder(folder)
    prompt = random_ids(cfg["vocab_size"], 9, 5)
    free_run = plain.greedy(prompt, 6, cfg, w)
    (folder / "generation_config.json").write_text(json.dumps({"eos_token_id": [free_run[2]]}))
    llm = LLM(folder, dtype="float32", max_seq_len=64)
    first_stop = free_run.index(free_run[2])
    out = llm.generate(prompt_token_ids=[prompt], sampling_params=SamplingParams(temperature=0.0, max_new_tokens=6))[0]
    assert out.finish_reason.value == "stop" and out.output_token_ids == free_run[:first_stop + 1]  # EOS included
    out = llm.generate(prompt_token_ids=[prompt], sampling_params=SamplingParams(temperature=0.0, max_new_tokens=6, ignore_eos=True))[0]
    assert out.finish_reason.value == "length" and out.output_token_ids == free_run
    # the context limit ends a request too
    long_prompt = random_ids(cfg["vocab_size"], 60, 6)
    out = llm.generate(prompt_token_ids=[long_prompt], sampling_params=SamplingParams(temperature=0.0, max_new_tokens=50, ignore_eos=True))[0]
    assert out.finish_reason.value == "length" and len(out.output_token_ids) == 4
    with pytest.raises(ValueError, match="does not fit"):
        llm.generate(prompt_token_ids=[random_ids(cfg["vocab_size"], 64, 7)])
    with pytest.raises(ValueError, match="exactly one"):
        llm.generate()
    with pytest.raises(ValueError, match="SamplingParams for"):
        llm.generate(prompt_token_ids=[prompt], sampling_params=[SamplingParams(), SamplingParams()])
    with pytest.raises(ValueError, match="tokenizer"):
        llm.generate("text without a tokenizer")


def test_seeded_sampling_is_reproducible_and_independent_of_batching(folders):
    from tokamak_amd import LLM, SamplingParams

    folder = folders["B"]
    cfg, _ = plain.read_folder(folder)
    prompts = [random_ids(cfg["vocab_size"], n, 90 + i) for i, n in enumerate([1, 9, 40, 70])]
    params = [SamplingParams(temperature=0.8, top_p=0.95, max_new_tokens=12, seed=100 + i, ignore_eos=True) for i in range(4)]
    llm = LLM(folder, dtype="float32", block_size=8, kv_pool_tokens=512, max_batch_size=4,
              max_num_batched_tokens=32, prefill_chunk=16)
    a = llm.generate(prompt_token_ids=prompts, sampling_params=params)
    b = llm.generate(prompt_token_ids=prompts, sampling_params=params)
    assert [o.output_token_ids for o in a] == [o.output_token_ids for o in b]
    alone = [llm.generate(prompt_token_ids=[p], sampling_params=q)[0] for p, q in zip(prompts, params)]
    assert [o.output_token_ids for o in a] == [o.output_token_ids for o in alone]
    other = llm.generate(prompt_token_ids=prompts, sampling_params=[
        SamplingParams(temperature=0.8, top_p=0.95, max_new_tokens=12, seed=7 + i, ignore_eos=True) for i in range(4)])
    assert [o.output_token_ids for o in a] != [o.output_token_ids for o in other]


def test_preemption_is_invisible(folders):
    """A pool of three pages for two requests (reference
    tests/integration/test_generate_e2e.py:180-213): outputs equal a roomy run."""
    from tokamak_amd import LLM, SamplingParams

    folder = folders["A"]
    cfg, _ = plain.read_folder(folder)
    prompts = [random_ids(cfg["vocab_size"], n, 20 + i) for i, n in enumerate([14, 13])]
    params = [SamplingParams(temperature=0.0, max_new_tokens=20, ignore_eos=True),
              SamplingParams(temperature=0.9, top_k=20, max_new_tokens=20, seed=3, ignore_eos=True)]
    roomy = LLM(folder, dtype="float32", max_seq_len=48, kv_pool_tokens=256, max_batch_size=2)
    tight = LLM(folder, dtype="float32", max_seq_len=48, kv_pool_tokens=48, max_batch_size=2)
    want = roomy.generate(prompt_token_ids=prompts, sampling_params=params)
    got = tight.generate(prompt_token_ids=prompts, sampling_params=params)
    assert tight.num_preemptions > 0 and roomy.num_preemptions == 0
    assert [o.output_token_ids for o in got] == [o.output_token_ids for o in want]
    tight.runner.manager.check()
    assert tight.runner.manager.num_free_pages() == 3


@pytest.mark.parametrize("which", ["A", "D"])
def test_random_workloads_do_not_depend_on_pool_budget_or_portions(tmp_path, which):
    """Random prompts and sampling parameters: a run with a tight page pool (so requests
    are preempted and recomputed), few running sequences, a small token budget and short
    prompt portions produces the tokens and finish reasons of a roomy run (float32)."""
    import random

    from tiny import TINIES, make_folder
    from tokamak_amd import LLM, SamplingParams

    folder = make_folder(tmp_path, which)
    cfg = TINIES[which]["config"]
    page, longest = TINIES[which]["page_size"], min(cfg.max_position_embeddings, 256)
    roomy = LLM(folder, dtype="float32", max_seq_len=longest, block_size=page, kv_pool_tokens=16 * longest,
                max_batch_size=16)
    preemptions = 0
    for seed in range(5):
        rng = random.Random(seed)
        count = rng.randint(2, 8)
        prompts = [[rng.randrange(cfg.vocab_size) for _ in range(rng.randint(1, longest // 2))] for _ in range(count)]
        params = [SamplingParams(temperature=rng.choice([0.0, 0.0, 0.8, 1.2]), top_k=rng.choice([0, 5, 40]),
                                 top_p=rng.choice([1.0, 0.9]), max_new_tokens=rng.randint(1, longest // 3),
                                 seed=rng.randrange(1 << 30), ignore_eos=rng.random() < 0.7) for _ in range(count)]
        want = roomy.generate(prompt_token_ids=prompts, sampling_params=params)
        tight = LLM(folder, dtype="float32", max_seq_len=longest, block_size=page,
                    kv_pool_tokens=longest + rng.randint(0, longest), max_batch_size=rng.randint(1, 6),
                    max_num_batched_tokens=rng.choice([8, 16, 64, 2048]), prefill_chunk=rng.choice([None, 2, 7, 16, 100]))
        got = tight.generate(prompt_token_ids=prompts, sampling_params=params)
        tight.runner.manager.check()
        preemptions += tight.num_preemptions
        assert [(o.output_token_ids, o.finish_reason) for o in got] == [(o.output_token_ids, o.finish_reason) for o in want]
    assert preemptions > 0


def test_typed_configuration_gives_the_weights_of_a_written_folder(tmp_path):
    """``LLM(config, seed=...)`` (random weights without a folder) generates what a
    folder written by ``write_random_model`` with the same seed generates."""
    from tiny import TINIES
    from tokamak_amd import LLM, SamplingParams
    from tokamak_amd.weights import write_random_model

    cfg = TINIES["B"]["config"]
    folder = write_random_model(tmp_path / "m", cfg, 5)
    prompts = [[3, 1, 4, 1, 5, 9, 2, 6], [7]]
    params = SamplingParams(temperature=0.0, max_new_tokens=10, ignore_eos=True)
    a = LLM(folder, dtype="float32", block_size=8).generate(prompt_token_ids=prompts, sampling_params=params)
    b = LLM(cfg, seed=5, dtype="float32", block_size=8).generate(prompt_token_ids=prompts, sampling_params=params)
    assert [o.output_token_ids for o in a] == [o.output_token_ids for o in b]
    c = LLM(cfg, seed=6, dtype="float32", block_size=8).generate(prompt_token_ids=prompts, sampling_params=params)
    assert [o.output_token_ids for o in a] != [o.output_token_ids for o in c]


def test_default_pool_holds_every_running_request_at_full_length(folders):
    from tokamak_amd import LLM

    llm = LLM(folders["A"], dtype="float32", max_seq_len=96, max_batch_size=5)
    assert llm.runner.kv_pool_tokens == 5 * 96
    assert llm.runner.manager.num_pages() == 5 * 96 // 16
    with pytest.raises(ValueError, match="kv_pool_tokens"):
        LLM(folders["A"], dtype="float32", max_seq_len=96, kv_pool_tokens=95)


def test_decode_batches_beyond_the_captured_size_run_eagerly(folders):
    """70 running sequences: decode steps of more than 64 tokens use the library product,
    which is kept out of HIP graphs; the tokens are those of running each prompt alone."""
    from tokamak_amd import LLM, SamplingParams

    folder = folders["D"]
    cfg, _ = plain.read_folder(folder)
    prompts = [random_ids(cfg["vocab_size"], 3 + i % 5, 300 + i) for i in range(70)]
    params = SamplingParams(temperature=0.0, max_new_tokens=4, ignore_eos=True)
    wide = LLM(folder, dtype="bfloat16", max_seq_len=32, max_batch_size=70)
    got = wide.generate(prompt_token_ids=prompts, sampling_params=params)
    assert not wide.runner._graphs                      # no step was captured
    narrow = LLM(folder, dtype="bfloat16", max_seq_len=32, max_batch_size=1)
    want = narrow.generate(prompt_token_ids=prompts[:6], sampling_params=params)
    assert narrow.runner._graphs
    same = sum(a.output_token_ids == b.output_token_ids for a, b in zip(got[:6], want))
    assert same >= 5                                    # bf16 rounding may flip a near tie


def test_command_line(folders, capsys):
    from tokamak_amd import cli

    assert cli.main(["--model", str(folders["A"]), "--prompt-ids", "5,6,7", "--max-new-tokens", "5",
                     "--temperature", "0", "--dtype", "float32", "--quiet"]) == 0
    out = capsys.readouterr().out
    assert "[completion (length)]" in out and "[prompt ids]" in out


def test_load_is_reported_and_progress_counts_finished_requests(folders, caplog, capsys):
    """What the reference reports (src/tokamak/engine/llm.py:180-189,299; model/loader.py:95): one
    line when loading starts, one with the number of tensors read, a bar over finished requests."""
    import logging

    from tokamak_amd import LLM, SamplingParams

    with caplog.at_level(logging.INFO, logger="tokamak_amd.engine.llm"):
        llm = LLM(folders["A"], dtype="float32", max_seq_len=64, max_batch_size=2)
    text = caplog.text
    assert "Loading" in text and "Qwen3ForCausalLM" in text and "float32" in text
    tensors = len(plain.read_folder(folders["A"])[1])
    assert f"Loaded {tensors} tensors" in text and "cache pool of 128 tokens" in text
    outs = llm.generate(prompt_token_ids=[[1, 2, 3], [4, 5], [6]],
                        sampling_params=SamplingParams(temperature=0.0, max_new_tokens=3, ignore_eos=True), use_tqdm=True)
    assert [len(o.output_token_ids) for o in outs] == [3, 3, 3]
    assert "Generating" in capsys.readouterr().err and "3/3" in llm.last_progress


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_captured_decode_steps_equal_eager_ones_on_every_replay(folders, dtype):
    """The same decode steps through replayed HIP graphs and eagerly, with the
    program's own eager work (prefill of other requests) and synchronisations
    between the replays; every replay is checked."""
    from tokamak_amd.engine.runner import ModelRunner, StepEntry

    folder = folders["C"]
    cfg, _ = plain.read_folder(folder)
    kw = dict(dtype=dtype, page_size=16, kv_pool_tokens=2048, max_requests=8)
    graphed = ModelRunner.from_folder(folder, use_graphs=True, **kw)
    eager = ModelRunner.from_folder(folder, use_graphs=False, **kw)
    prompts = {r: random_ids(cfg["vocab_size"], n, 300 + r) for r, n in enumerate([30, 7, 250])}
    last = {}
    for r, p in prompts.items():
        a = graphed.step([StepEntry(r, p, [len(p) - 1])])
        b = eager.step([StepEntry(r, p, [len(p) - 1])])
        assert torch.equal(a, b)
        last[r] = int(a.argmax())
    for i in range(40):
        if i == 7:      # a newcomer's prefill between replays, and a request that ends
            p = random_ids(cfg["vocab_size"], 19, 999)
            a = graphed.step([StepEntry(9, p, [18])])
            b = eager.step([StepEntry(9, p, [18])])
            assert torch.equal(a, b)
            last[9] = int(a.argmax())
        if i == 20:
            graphed.end(1)
            eager.end(1)
            del last[1]
        entries = [StepEntry(r, [t], [0]) for r, t in last.items()]
        a = graphed.step(entries).clone()
        torch.cuda.synchronize()
        b = eager.step(entries)
        assert torch.equal(a, b), f"replay {i} differs from the eager step"
        for row, r in enumerate(list(last)):
            last[r] = int(a[row].argmax())
    assert len(graphed._graphs) >= 2     # batch sizes 3, 4 and 3 again; lengths crossing 256
    # the step that meets a new shape runs eagerly and is recorded; every later one is a replay
    assert sum(g.replays for g in graphed._graphs.values()) == 40 - len(graphed._graphs)


def test_nothing_is_garbage_collected_while_a_step_is_recorded(folders):
    """Cyclic garbage that owns GPU objects of its own (an older runner's recorded steps) may not
    be destroyed in the middle of a recording: the HIP runtime ends the process when a recorded
    step is destroyed then.  Collection is therefore off while a step is recorded.  Here every
    allocation would start a collection (threshold 1), an older runner with recorded steps is
    garbage in a cycle, and a new runner records a step: no collection starts while the stream
    is being recorded, and the step gives the eager runner's logits."""
    import gc

    from tokamak_amd.engine.runner import ModelRunner, StepEntry

    folder = folders["C"]
    cfg, _ = plain.read_folder(folder)
    kw = dict(dtype="bfloat16", page_size=16, kv_pool_tokens=512, max_requests=4)
    prompt = random_ids(cfg["vocab_size"], 20, 5)

    old = ModelRunner.from_folder(folder, use_graphs=True, **kw)
    old.step([StepEntry("a", prompt, [])])
    for token in (3, 4, 5):
        old.step([StepEntry("a", [token], [0])])
    assert old._graphs and sum(g.replays for g in old._graphs.values()) >= 2
    old.myself = old            # only a collection can free it now
    del old

    new = ModelRunner.from_folder(folder, use_graphs=True, **kw)
    eager = ModelRunner.from_folder(folder, use_graphs=False, **kw)
    for runner in (new, eager):
        runner.step([StepEntry("a", prompt, [])])
    during = []

    def watch(phase, info):
        if phase == "start" and torch.cuda.is_current_stream_capturing():
            during.append(info)

    threshold = gc.get_threshold()
    gc.callbacks.append(watch)
    gc.set_threshold(1, 1, 1)
    try:
        got = [new.step([StepEntry("a", [token], [0])]).clone() for token in (3, 4, 5)]
    finally:
        gc.set_threshold(*threshold)
        gc.callbacks.remove(watch)
    assert new._graphs and not during, "a collection started while a step was being recorded"
    assert gc.isenabled()
    for token, have in zip((3, 4, 5), got):
        assert torch.equal(have, eager.step([StepEntry("a", [token], [0])]))
    gc.collect()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_captured_decode_steps_queued_without_a_host_sync(folders, dtype):
    """Forced tokens, nothing wanted, no synchronisation between steps: the host packs
    descriptor N+1 while the copy of descriptor N may still be queued behind the running
    graph.  Each descriptor must reach the graph it was packed for: the logits after 24
    such steps equal the eager runner's, and so does every key that was cached."""
    from tokamak_amd.engine.runner import ModelRunner, StepEntry

    folder = folders["C"]
    cfg, _ = plain.read_folder(folder)
    kw = dict(dtype=dtype, page_size=16, kv_pool_tokens=1024, max_requests=4)
    graphed = ModelRunner.from_folder(folder, use_graphs=True, **kw)
    eager = ModelRunner.from_folder(folder, use_graphs=False, **kw)
    prompts = {r: random_ids(cfg["vocab_size"], n, 70 + r) for r, n in enumerate([21, 5, 40])}
    forced = {r: random_ids(cfg["vocab_size"], 25, 80 + r) for r in prompts}
    for runner in (graphed, eager):
        for r, p in prompts.items():
            runner.step([StepEntry(r, p, [])])
    # make the device slow to reach the copies: a long eager step of another request first
    filler = random_ids(cfg["vocab_size"], 600, 99)
    graphed.step([StepEntry("filler", filler, [])])
    for i in range(24):
        graphed.step([StepEntry(r, [forced[r][i]], []) for r in prompts])
    a = graphed.step([StepEntry(r, [forced[r][24]], [0]) for r in prompts]).clone()
    for i in range(24):
        eager.step([StepEntry(r, [forced[r][i]], []) for r in prompts])
    b = eager.step([StepEntry(r, [forced[r][24]], [0]) for r in prompts])
    assert torch.equal(a, b)
    assert sum(g.replays for g in graphed._graphs.values()) >= 20
    for slot in range(cfg["num_hidden_layers"]):
        for name in ("k", "v"):
            ga, ea = graphed.storage.slot(slot).arrays[name], eager.storage.slot(slot).arrays[name]
            for r in prompts:
                pages_g = graphed.manager.block_table(r)
                pages_e = eager.manager.block_table(r)
                assert torch.equal(ga[pages_g], ea[pages_e])


@pytest.mark.parametrize("use_graphs", [False, True], ids=["eager", "replayed"])
def test_a_step_takes_tokens_that_are_still_on_the_gpu(folders, use_graphs):
    """``StepEntry.feed``: a decode token named by its row in the sampler's output instead
    of by its value gives the logits of the same step with the value given, in steps that
    are replayed from a recording and in steps that are not, beside entries whose tokens
    the host gives; and what it refuses."""
    from tokamak_amd.engine.runner import ModelRunner, StepEntry

    folder = folders["E"] if "E" in folders else folders["A"]
    cfg, _ = plain.read_folder(folder)
    prompts = [random_ids(cfg["vocab_size"], n, 60 + i) for i, n in enumerate([9, 21, 5])]
    nxt = [random_ids(cfg["vocab_size"], 6, 80 + i) for i in range(3)]

    def run(fed):
        runner = ModelRunner.from_folder(folder, dtype="bfloat16", page_size=16, kv_pool_tokens=256, max_requests=4,
                                         use_graphs=use_graphs)
        for r, p in enumerate(prompts):
            runner.step([StepEntry(r, p, [])])
        out = []
        for i in range(6):
            if fed:
                # rows in another order than the entries, as a sampler might leave them
                runner.sampled[:4].copy_(torch.tensor([nxt[2][i], 0, nxt[0][i], nxt[1][i]], dtype=torch.int32))
                entries = [StepEntry(0, [0], [0], feed=2), StepEntry(1, [nxt[1][i]], [0]), StepEntry(2, [0], [0], feed=0)]
            else:
                entries = [StepEntry(r, [nxt[r][i]], [0]) for r in range(3)]
            if i == 3:      # a prompt portion beside them: a step that is not replayed
                entries.append(StepEntry(3, random_ids(cfg["vocab_size"], 7, 99), [6]))
            out.append(runner.step(entries).cpu())
        assert bool(runner._graphs) == use_graphs
        return runner, out

    _, want = run(False)
    runner, got = run(True)
    for i, (a, b) in enumerate(zip(want, got)):
        assert torch.equal(a, b), f"step {i}"
    with pytest.raises(ValueError):
        runner.step([StepEntry(0, [1, 2], [0], feed=0)])
    with pytest.raises(ValueError):
        runner.step([StepEntry(0, [1], [0], feed=4)])
    runner.manager.check()


@pytest.mark.parametrize("which", ["A", "D"])
def test_running_one_step_ahead_changes_no_token(tmp_path, which):
    """The step loop launches a step before it has read the tokens of the step before.
    Random workloads (greedy and sampled, stops on EOS ids that do occur and on length,
    tight pools with preemption, small budgets): tokens and finish reasons equal those of
    a loop that reads every step's tokens before it plans the next."""
    import json
    import random

    from tokamak_amd import LLM, SamplingParams

    folder = make_folder(tmp_path, which)
    cfg = TINIES[which]["config"]
    page, longest = TINIES[which]["page_size"], min(cfg.max_position_embeddings, 256)
    # ids that greedy runs of this model do produce, so that some requests stop on them
    probe = LLM(folder, dtype="float32", max_seq_len=longest, block_size=page, kv_pool_tokens=4 * longest, max_batch_size=4)
    seen = probe.generate(prompt_token_ids=[[3, 1, 4], [1, 5, 9, 2, 6]],
                          sampling_params=SamplingParams(temperature=0.0, max_new_tokens=30, ignore_eos=True))
    eos = sorted({o.output_token_ids[7] for o in seen} | {o.output_token_ids[20] for o in seen})
    (folder / "generation_config.json").write_text(json.dumps({"eos_token_id": eos}))
    stops = preemptions = 0
    for seed in range(6):
        rng = random.Random(100 + seed)
        count = rng.randint(2, 8)
        prompts = [[rng.randrange(cfg.vocab_size) for _ in range(rng.randint(1, longest // 2))] for _ in range(count)]
        prompts[0] = [3, 1, 4]
        params = [SamplingParams(temperature=rng.choice([0.0, 0.0, 0.8, 1.2]), top_k=rng.choice([0, 5, 40]),
                                 top_p=rng.choice([1.0, 0.9]), max_new_tokens=rng.randint(1, longest // 3),
                                 seed=rng.randrange(1 << 30), ignore_eos=rng.random() < 0.3) for _ in range(count)]
        params[0] = SamplingParams(temperature=0.0, max_new_tokens=30)
        kwargs = dict(dtype="float32", max_seq_len=longest, block_size=page, kv_pool_tokens=longest + rng.randint(0, longest),
                      max_batch_size=rng.randint(1, 6), max_num_batched_tokens=rng.choice([8, 16, 64, 2048]),
                      prefill_chunk=rng.choice([None, 2, 7, 16, 100]))
        ahead = LLM(folder, steps_ahead=True, **kwargs)
        in_turn = LLM(folder, steps_ahead=False, **kwargs)
        got = ahead.generate(prompt_token_ids=prompts, sampling_params=params)
        want = in_turn.generate(prompt_token_ids=prompts, sampling_params=params)
        assert [(o.output_token_ids, o.finish_reason) for o in got] == [(o.output_token_ids, o.finish_reason) for o in want]
        for llm in (ahead, in_turn):
            llm.runner.manager.check()
            assert llm.runner.manager.num_free_pages() == llm.runner.manager.num_pages()
        stops += sum(o.finish_reason.value == "stop" for o in got)
        preemptions += ahead.num_preemptions
    assert stops > 0 and preemptions > 0
