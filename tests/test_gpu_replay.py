"""Trace replay through bin/trace_run, in float32 and bfloat16: each request
alone and whole; most of it in one step and the last 32 tokens one by one;
portions of changing size down to two tokens; and mixed, up to four live
requests with so few pages that they are used again.  Everything is compared
with the plain implementation run on whole sequences."""

import pytest

from replay_util import TOL, compare, expected_logits, mixed, portions, random_ids, run_trace, tail_one_by_one, whole
from tiny import TINIES, make_folder

pytestmark = pytest.mark.gpu

LENGTHS = {"A": [5, 17, 33, 100, 128], "B": [1, 9, 40, 70, 201], "C": [2, 31, 64, 130, 77]}


@pytest.fixture(scope="module")
def setups(tmp_path_factory):
    root = tmp_path_factory.mktemp("replay")
    out = {}
    for which in LENGTHS:
        folder = make_folder(root, which)
        vocab = TINIES[which]["config"].vocab_size
        requests = {f"r{i}": random_ids(vocab, n, 100 + i) for i, n in enumerate(LENGTHS[which])}
        out[which] = (folder, requests, expected_logits(folder, requests))
    return out


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["A", "B", "C"])
def test_replay_all_cuttings(setups, tmp_path, which, dtype):
    folder, requests, expected = setups[which]
    ps = TINIES[which]["page_size"]
    longest = max(len(t) for t in requests.values())
    # one process replays: whole, tail one by one, portions (one request live at a time)
    steps = []

    def add(more):
        base = len(steps)
        for rec in more:
            steps.append(dict(rec, step=base + rec["step"]))

    add(whole(requests))
    for rid, toks in requests.items():
        add(tail_one_by_one(rid, toks))
        add(portions(rid, toks))
    got = run_trace(folder, dtype, steps, max_tokens=-(-longest // 64) * 64, out_dir=tmp_path / "o1", page_size=ps)
    # the three cuttings visit every request three times: compare each pass
    worst = 0.0
    at = 0
    for block in [whole(requests)] + [f(rid, toks) for rid, toks in requests.items() for f in (tail_one_by_one, portions)]:
        part = steps[at:at + len(block)]
        at += len(block)
        worst = max(worst, compare(part, got, expected, **TOL[dtype]))
    print(f"{which} {dtype}: worst error over whole/tail/portions {worst:.3e}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["A", "B", "C"])
def test_replay_mixed_with_page_reuse(setups, tmp_path, which, dtype):
    folder, requests, expected = setups[which]
    vocab = TINIES[which]["config"].vocab_size
    # eight requests so that later ones run in pages the first ones gave back
    more = dict(requests)
    for i, n in enumerate([23, 64, 49]):
        more[f"s{i}"] = random_ids(vocab, n, 500 + i)
    exp = dict(expected)
    exp.update(expected_logits(folder, {k: v for k, v in more.items() if k not in expected}))
    steps, peak = mixed(more, seed=11)
    assert max(len(s["entries"]) for s in steps) >= 3
    got = run_trace(folder, dtype, steps, max_tokens=peak, out_dir=tmp_path / "o2", page_size=TINIES[which]["page_size"])
    worst = compare(steps, got, exp, **TOL[dtype])
    print(f"{which} {dtype}: mixed, {len(steps)} steps, pool {peak} tokens, worst error {worst:.3e}")
