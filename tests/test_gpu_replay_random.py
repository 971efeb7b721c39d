"""Random traces through the engine's step function (the one ``bin/trace_run`` drives)
on small models whose head and page sizes are those of the matrix-core attention
kernels: random request lengths, up to four live requests cut at random into
portions beside single tokens, a page pool with no slack so that pages are used
again, float32 and bfloat16, every wanted row against the plain implementation."""

import random

import pytest

import plain_qwen3 as plain
from replay_util import TOL, compare, mixed
from tiny import TINIES, make_folder

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["D", "E", "F"])
def test_random_traces_match_plain(tmp_path, which, dtype):
    from tokamak_amd.engine.runner import ModelRunner, StepEntry

    folder = make_folder(tmp_path, which)
    cfg_json, weights = plain.read_folder(folder)
    vocab = cfg_json["vocab_size"]
    worst = 0.0
    for seed in range(6):
        rng = random.Random(1000 * seed + len(which))
        lengths = [rng.choice([1, 2, 17, 40, 70, 130, 200, 333]) + rng.randint(0, 15) for _ in range(rng.randint(3, 6))]
        requests = {f"r{i}": [rng.randrange(vocab) for _ in range(n)] for i, n in enumerate(lengths)}
        steps, peak = mixed(requests, seed, max_live=4, tail=rng.choice([0, 3, 6, 20]))
        page = TINIES[which]["page_size"]
        runner = ModelRunner.from_folder(folder, dtype=dtype, page_size=page, kv_pool_tokens=max(peak, page),
                                         max_requests=4)
        got = {}
        for rec in steps:
            out = runner.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in rec["entries"]])
            if out.shape[0]:
                got[rec["step"]] = out.cpu().numpy().copy()
            for request in rec["end"]:
                runner.end(request)
        runner.manager.check()
        expected = {rid: plain.logits(toks, cfg_json, weights).numpy() for rid, toks in requests.items()}
        worst = max(worst, compare(steps, got, expected, **TOL[dtype]))
    print(f"tiny {which} {dtype}: worst error {worst:.2e}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_long_request_in_small_portions_beside_short_ones(tmp_path, dtype):
    """1,500 tokens fed in portions of at most 40 beside three short requests: late
    portions are a few tiles over more than a thousand keys, which the bfloat16
    attention kernel cuts into pieces and merges."""
    from tokamak_amd.engine.runner import ModelRunner, StepEntry

    folder = make_folder(tmp_path, "F")
    cfg_json, weights = plain.read_folder(folder)
    rng = random.Random(5)
    requests = {name: [rng.randrange(cfg_json["vocab_size"]) for _ in range(n)]
                for name, n in [("long", 1500), ("a", 33), ("b", 70), ("c", 5)]}
    steps, peak = mixed(requests, 3, max_live=4, tail=4)
    runner = ModelRunner.from_folder(folder, dtype=dtype, page_size=16, kv_pool_tokens=peak, max_requests=4)
    got = {}
    for rec in steps:
        out = runner.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in rec["entries"]])
        if out.shape[0]:
            got[rec["step"]] = out.cpu().numpy().copy()
        for request in rec["end"]:
            runner.end(request)
    runner.manager.check()
    expected = {rid: plain.logits(toks, cfg_json, weights).numpy() for rid, toks in requests.items()}
    print(f"{dtype}: {len(steps)} steps, worst error {compare(steps, got, expected, **TOL[dtype]):.2e}")
