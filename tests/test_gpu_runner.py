"""The step function's own bookkeeping: a step that cannot run leaves nothing behind,
generation gives back what its scheduler reserved when a step fails, and captured
decode shapes stay within their memory."""

import pytest
import torch

import plain_qwen3 as plain
from replay_util import random_ids
from tiny import TINIES, make_folder

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def folder(tmp_path_factory):
    return make_folder(tmp_path_factory.mktemp("runner"), "A")


def test_a_step_that_cannot_run_changes_nothing(folder):
    from tokamak_amd.cache import OutOfPagesError
    from tokamak_amd.cache.manager import OutOfSlotsError
    from tokamak_amd.engine.runner import ModelRunner, StepEntry

    runner = ModelRunner.from_folder(folder, dtype="float32", page_size=16, kv_pool_tokens=96, max_requests=3)
    manager = runner.manager
    runner.step([StepEntry("old", random_ids(256, 30, 1), [])])          # 2 of 6 pages
    before = (manager.num_free_pages(), manager.slots.num_free, dict(runner._ctx_len))

    def unchanged():
        manager.check()
        assert (manager.num_free_pages(), manager.slots.num_free, dict(runner._ctx_len)) == before
        assert manager.block_table("new") == [] and not runner.is_live("new")

    # the first entry alone would fit; the second does not: neither gets anything
    with pytest.raises(OutOfPagesError, match="needs 6 more page"):
        runner.step([StepEntry("new", [1] * 40, []), StepEntry("big", [2] * 33, [])])
    unchanged()
    with pytest.raises(ValueError, match="token id outside"):
        runner.step([StepEntry("new", [1, 2, 3], []), StepEntry("old", [256], [0])])
    unchanged()
    with pytest.raises(ValueError, match="the model's limit is 128"):
        runner.step([StepEntry("new", [1, 2, 3], []), StepEntry("old", [5] * 99, [0])])
    unchanged()
    with pytest.raises(ValueError, match="appears twice"):
        runner.step([StepEntry("new", [1], []), StepEntry("new", [2], [])])
    unchanged()
    with pytest.raises(ValueError, match="wants logits outside"):
        runner.step([StepEntry("new", [1, 2], [2])])
    unchanged()
    with pytest.raises(OutOfSlotsError, match="3 new request"):
        runner.step([StepEntry(("n", i), [1], []) for i in range(3)])
    unchanged()
    # and the runner still works: the old request goes on where it was
    ids = random_ids(256, 30, 1)
    cfg, w = plain.read_folder(folder)
    got = runner.step([StepEntry("old", [7], [0])]).cpu()
    torch.testing.assert_close(got[0], plain.logits(ids + [7], cfg, w)[-1], rtol=0, atol=5e-5)


def test_generation_that_fails_midway_gives_everything_back(folder, monkeypatch):
    from tokamak_amd import LLM, SamplingParams

    llm = LLM(folder, dtype="float32", kv_pool_tokens=128, max_batch_size=2, max_num_batched_tokens=16)
    prompts = [random_ids(256, n, 20 + i) for i, n in enumerate([40, 9, 25, 14])]
    params = SamplingParams(temperature=0.0, max_new_tokens=5, ignore_eos=True)
    good = [o.output_token_ids for o in llm.generate(prompt_token_ids=prompts, sampling_params=params)]

    real_step, calls = llm.runner.step, []

    def failing_step(entries):
        calls.append(len(entries))
        if len(calls) == 4:                 # portions reserved, some requests running, others waiting
            raise RuntimeError("injected failure")
        return real_step(entries)

    monkeypatch.setattr(llm.runner, "step", failing_step)
    with pytest.raises(RuntimeError, match="injected failure"):
        llm.generate(prompt_token_ids=prompts, sampling_params=params)
    manager = llm.runner.manager
    manager.check()
    assert manager.num_free_pages() == manager.num_pages() and manager.slots.num_free == 2
    assert all(t == [] for t in (manager.block_table(i) for i in range(4)))
    monkeypatch.setattr(llm.runner, "step", real_step)
    again = [o.output_token_ids for o in llm.generate(prompt_token_ids=prompts, sampling_params=params)]
    assert again == good                    # request ids start at 0 again and meet no leftovers


def test_captured_shapes_are_dropped_to_stay_within_their_memory(folder):
    from tokamak_amd.engine.runner import ModelRunner, StepEntry

    kw = dict(dtype="bfloat16", page_size=16, kv_pool_tokens=512, max_requests=8)
    probe = ModelRunner.from_folder(folder, **kw)
    probe.step([StepEntry(0, [1, 2, 3], [])])
    probe.step([StepEntry(0, [4], [0])])
    one = next(iter(probe._graphs.values())).bytes
    assert one > 0
    capped = ModelRunner.from_folder(folder, graph_memory_bytes=int(2.5 * one), **kw)
    eager = ModelRunner.from_folder(folder, use_graphs=False, **kw)
    for runner in (capped, eager):
        runner.step([StepEntry(r, random_ids(256, 3 + r, r), []) for r in range(8)])
    for live in (8, 7, 6, 5, 8, 7, 6, 5, 4, 3):          # shapes come back after they were dropped
        entries = [StepEntry(r, [9 + live], [0]) for r in range(live)]
        a = capped.step(entries).clone()
        b = eager.step(entries)
        assert torch.equal(a, b)
        assert sum(g.bytes for g in capped._graphs.values()) <= 2.5 * one or len(capped._graphs) == 1
    assert 1 <= len(capped._graphs) <= 2
