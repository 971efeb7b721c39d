"""Schedules and sizes that generation reaches but the replay traces do not: decode
steps of more than 64 requests (beyond the captured and the weight-streaming
kernels: eager, library products, the head read once per 64 rows); long portions of
two requests beside decode tokens of others at Qwen3-32B's width; the full
vocabulary's head; all 36 layers of Qwen3-8B's width.  Every compared row is a row of
logits against the plain implementation, never an agreement of tokens."""

import dataclasses

import pytest
import torch

import plain_qwen3 as plain
from replay_util import random_ids
from tiny import TINIES
from tokamak_amd.config import find_preset, get_architecture

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


class LazyWeights(dict):
    """name -> float32 CPU tensor, drawn when asked for (a model of tens of gigabytes
    never sits in host memory whole).  The same source feeds the engine."""

    def __init__(self, source):
        super().__init__()
        self.source = source

    def __getitem__(self, name):
        return self.source.fetch(name).to("cpu", torch.float32)

    def __contains__(self, name):
        return name in self.source.expected


def shaped(preset, *, on_gpu, seed=3, jitter=0.1, **changes):
    """(typed config, config.json dict, plan, weight source, plain weights) of a preset's
    widths with some sizes replaced."""
    from tokamak_amd.weights.random_init import expected_tensors_of
    from tokamak_amd.weights.sources import RandomSource

    arch, full = find_preset(preset)
    cfg = dataclasses.replace(full, **changes)
    plan = arch.plan(cfg)
    expected = {n: s for n, s in expected_tensors_of(plan).items() if not s.ignored}
    source = RandomSource(expected, seed=seed, matrix_std=0.02, vector_jitter=jitter, dtype=torch.bfloat16,
                          device=DEV if on_gpu else "cpu")
    return cfg, arch.to_json(cfg), plan, source, LazyWeights(source)


def tolerance(dtype, want):
    return 5e-5 if dtype == "float32" else 2e-3 + 2e-2 * float(want.abs().max())


def decode_rows_against_plain(plan, source, cfg_json, w, dtype, lengths, page_size, vocab):
    """Prefill ``len(lengths)`` requests a few at a time, then ONE step that brings one
    token of every request; each row of its logits against the plain implementation."""
    from tokamak_amd.engine.runner import ModelRunner, StepEntry

    n = len(lengths)
    runner = ModelRunner(plan, source, dtype=dtype, page_size=page_size,
                         kv_pool_tokens=sum(-(-(t + 1) // page_size) * page_size for t in lengths),
                         max_requests=n)
    prompts = [random_ids(vocab, t + 1, 500 + i) for i, t in enumerate(lengths)]     # the last token decodes
    for at in range(0, n, 16):
        runner.step([StepEntry(r, prompts[r][:-1], []) for r in range(at, min(at + 16, n))])
    got = runner.step([StepEntry(r, [prompts[r][-1]], [0]) for r in range(n)]).cpu()
    assert got.shape == (n, vocab)
    worst = 0.0
    for r in range(n):
        want = plain.logits(prompts[r], cfg_json, w)[-1]
        err = float((got[r] - want).abs().max())
        assert err <= tolerance(dtype, want), f"request {r} of {n} ({lengths[r]} cached tokens): {err}"
        worst = max(worst, err)
    runner.manager.check()
    return worst


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_decode_step_of_a_hundred_requests_tiny(tmp_path, dtype):
    from tiny import make_folder
    from tokamak_amd.config import load_model_description
    from tokamak_amd.weights.sources import SafetensorsSource

    folder = make_folder(tmp_path, "D")
    _, _, plan = load_model_description(folder)
    cfg_json, w = plain.read_folder(folder)
    lengths = [1 + (7 * i) % 45 for i in range(100)]
    worst = decode_rows_against_plain(plan, SafetensorsSource(folder), cfg_json, w, dtype, lengths,
                                      TINIES["D"]["page_size"], cfg_json["vocab_size"])
    print(f"{dtype}: 100 decode rows, worst {worst:.2e}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_decode_step_of_eighty_requests_at_8b_width(dtype):
    cfg, cfg_json, plan, source, w = shaped("qwen3-8b", on_gpu=False, num_layers=2, vocab_size=8192,
                                            max_position_embeddings=4096)
    weights = {n: source.fetch(n) for n in source.expected}          # drawn once, on the CPU

    class Fixed:
        expected = source.expected

        def names(self):
            return source.names()

        def fetch(self, name):
            return weights[name]

    lengths = [3 + (5 * i) % 20 for i in range(80)]
    worst = decode_rows_against_plain(plan, Fixed(), cfg_json, LazyWeights(Fixed()), dtype, lengths, 16, cfg.vocab_size)
    print(f"{dtype}: 80 decode rows at width {cfg.hidden_size}, worst {worst:.2e}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_portions_beside_decode_tokens_at_32b_width(dtype):
    """The schedule of 32 long prompts cut at 2,048 tokens beside running requests, in
    small: one step holds a 2,048-token portion from the start of one request, a
    2,048-token portion from the middle of another, and one decode token each of two
    short requests; the next step their rest.  One layer of Qwen3-32B's width."""
    from tokamak_amd.engine.runner import ModelRunner, StepEntry

    cfg, cfg_json, plan, source, w = shaped("qwen3-32b", on_gpu=True, num_layers=1, vocab_size=4096,
                                            max_position_embeddings=8192)
    runner = ModelRunner(plan, source, dtype=dtype, page_size=16, kv_pool_tokens=6144, max_requests=4)
    x = random_ids(cfg.vocab_size, 2100, 1)          # from its start
    y = random_ids(cfg.vocab_size, 2049 + 300, 2)    # from position 300
    p = random_ids(cfg.vocab_size, 25, 3)
    q = random_ids(cfg.vocab_size, 9, 4)
    runner.step([StepEntry("y", y[:300], []), StepEntry("p", p[:-2], []), StepEntry("q", q[:-2], [])])
    first = runner.step([StepEntry("p", [p[-2]], [0]), StepEntry("x", x[:2048], [2047]),
                         StepEntry("q", [q[-2]], [0]), StepEntry("y", y[300:2348], [0, 2047])]).cpu()
    second = runner.step([StepEntry("x", x[2048:], [51]), StepEntry("p", [p[-1]], [0]),
                          StepEntry("y", [y[2348]], [0]), StepEntry("q", [q[-1]], [0])]).cpu()
    want = {k: plain.logits(v, cfg_json, w) for k, v in (("x", x), ("y", y), ("p", p), ("q", q))}
    rows = [("p decode", first[0], want["p"][-2]), ("x portion end", first[1], want["x"][2047]),
            ("q decode", first[2], want["q"][-2]), ("y portion start", first[3], want["y"][300]),
            ("y portion end", first[4], want["y"][2347]), ("x short portion", second[0], want["x"][2099]),
            ("p decode 2", second[1], want["p"][-1]), ("y decode after portion", second[2], want["y"][2348]),
            ("q decode 2", second[3], want["q"][-1])]
    for what, got, ref in rows:
        err = float((got - ref).abs().max())
        print(f"{dtype} {what}: {err:.2e}")
        assert err <= tolerance(dtype, ref), what


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_head_over_the_full_vocabulary(dtype):
    """8 rows of [8, 4096] x [151936, 4096]^T through the head part, against float64."""
    from tokamak_amd.config import get_part

    V, H = 151936, 4096
    g = torch.Generator().manual_seed(0)
    table = (torch.randn(V, H, generator=g) * 0.02).to(dtype)
    h = torch.randn(8, H, generator=g).to(dtype)
    head = get_part("head", "linear_head")(vocab_size=V, dim=H, tied=False, dtype=dtype, device=DEV)
    head.bind("h.", lambda name: table.to(DEV))
    got = head.forward(h.to(DEV)).cpu()
    assert got.shape == (8, V) and got.dtype == torch.float32
    worst = 0.0
    for at in range(0, V, 16384):                                  # float64 a slab at a time
        want = h.double() @ table[at:at + 16384].double().T
        worst = max(worst, float((got[:, at:at + 16384].double() - want).abs().max()))
    scale = float(got.abs().max())
    print(f"{dtype}: full-vocabulary logits, worst {worst:.2e} at scale {scale:.2f}")
    # float32: 4096 products of magnitude 0.02 summed in pieces: 1e-5 is 40 ulp of the result.
    # bfloat16 inputs are exact here (the reference is computed from the same rounded values);
    # what is left is the float32 accumulation in another order.
    assert worst < 2e-5


def test_all_36_layers_of_8b_width_in_float32():
    """Depth: the whole stack of Qwen3-8B-shaped layers in true 32-bit, a 64-token
    prompt whole and its last 8 tokens one by one (captured steps), every position's
    logits against the plain implementation.  The vocabulary is cut to 8,192 (the full
    one is covered above); weights are drawn on the GPU and fetched layer by layer for
    the plain side."""
    from tokamak_amd.engine.runner import ModelRunner, StepEntry

    cfg, cfg_json, plan, source, w = shaped("qwen3-8b", on_gpu=True, vocab_size=8192, max_position_embeddings=4096)
    assert cfg.num_layers == 36 and len(plan.order) == 36
    runner = ModelRunner(plan, source, dtype="float32", page_size=16, kv_pool_tokens=256, max_requests=2)
    ids = random_ids(cfg.vocab_size, 64, 11)
    want = plain.logits(ids, cfg_json, w)
    whole = runner.step([StepEntry("a", ids, list(range(64)))]).cpu()
    runner.end("a")
    rows = [runner.step([StepEntry("a", ids[:56], list(range(56)))]).cpu()]
    for t in ids[56:]:
        rows.append(runner.step([StepEntry("a", [t], [0])]).cpu().clone())
    scale = float(want.abs().max())
    e1, e2 = float((whole - want).abs().max()), float((torch.cat(rows) - want).abs().max())
    print(f"36 layers float32: logit scale {scale:.2f}; whole {e1:.2e}; tail one by one {e2:.2e}")
    assert e1 < 2e-4 and e2 < 2e-4      # 36 layers deep: four times the two-layer bound


def test_32b_width_default_pool_leaves_room_for_steps_and_graphs():
    """Construction as generation does it (pool sized from free memory, 64 requests)
    with memory_fraction 0.97 and no other cap: after the pool is taken, a 2,048-token
    step and 64 captured decode shapes must still find their memory.  2 of the 64
    layers of Qwen3-32B's shape."""
    from tokamak_amd.engine.runner import ModelRunner, StepEntry

    cfg, _, plan, source, _ = shaped("qwen3-32b", on_gpu=True, jitter=0.0, num_layers=2, max_position_embeddings=8192)
    free_before, total = torch.cuda.mem_get_info()
    runner = ModelRunner(plan, source, dtype="bfloat16", page_size=16, kv_pool_tokens=None, max_requests=64,
                         tokens_per_request=10 ** 8, memory_fraction=0.97, max_step_tokens=2048)
    free_after, _ = torch.cuda.mem_get_info()
    print(f"pool of {runner.kv_pool_tokens} tokens ({runner.storage.bytes() / 2**30:.1f} GiB); measured step memory "
          f"{runner.step_memory_bytes / 2**20:.0f} MiB; graph budget {runner.graph_memory_bytes / 2**30:.0f} GiB; "
          f"free {free_before / 2**30:.1f} -> {free_after / 2**30:.1f} GiB of {total / 2**30:.1f}")
    assert runner.step_memory_bytes > 64 * cfg.vocab_size * 4          # at least the logits of 64 rows
    assert runner.storage.bytes() > 0.5 * free_before                  # the pool did take what there was
    prompts = [random_ids(cfg.vocab_size, 5 + r, r) for r in range(64)]
    for at in range(0, 64, 16):
        runner.step([StepEntry(r, prompts[r], []) for r in range(at, at + 16)])
    for live in range(64, 0, -1):                                       # 64 batch sizes, 64 captured shapes
        logits = runner.step([StepEntry(r, [1], [0]) for r in range(live)])
        assert logits.shape == (live, cfg.vocab_size)
        runner.end(live - 1)
    assert len(runner._graphs) == 64
    assert sum(g.bytes for g in runner._graphs.values()) <= runner.graph_memory_bytes
    long = random_ids(cfg.vocab_size, 2048, 99)
    out = runner.step([StepEntry("long", long, [2047])])
    assert torch.isfinite(out).all()
    torch.cuda.synchronize()


@pytest.mark.parametrize("use_graphs", [False, True], ids=["eager", "replayed"])
def test_decode_steps_of_few_requests_over_deep_contexts_at_8b_width(use_graphs, monkeypatch):
    """bfloat16 decode steps of three requests that hold 40, 700 and 2,300 tokens, at
    Qwen3-8B's width: the steps in which the o projection adds into the residual stream
    itself, the gate/up product finishes the norm after it, and the attention kernel makes
    its own queries and keys.  Eight steps, eager and replayed from a recorded step; every
    row of logits against the plain implementation."""
    from tokamak_amd.engine.runner import ModelRunner, StepEntry
    from tokamak_amd.kernels import ops

    cfg, cfg_json, plan, source, w = shaped("qwen3-8b", on_gpu=True, num_layers=2, vocab_size=4096,
                                            max_position_embeddings=4096)
    lengths = [40, 700, 2300]
    steps = 8
    calls = {"added": 0, "scaled": 0}
    add, gated = ops.gemm_wholek_add, ops.gemm_stream_swiglu

    def watched_add(*args, **kwargs):
        calls["added"] += 1
        return add(*args, **kwargs)

    def watched_gated(*args, **kwargs):
        calls["scaled"] += kwargs.get("sumsq") is not None
        return gated(*args, **kwargs)

    monkeypatch.setattr(ops, "gemm_wholek_add", watched_add)
    monkeypatch.setattr(ops, "gemm_stream_swiglu", watched_gated)
    runner = ModelRunner(plan, source, dtype="bfloat16", page_size=16, kv_pool_tokens=3200, max_requests=3,
                         use_graphs=use_graphs)
    ids = [random_ids(cfg.vocab_size, t + steps, 40 + i) for i, t in enumerate(lengths)]
    for r, t in enumerate(lengths):
        for at in range(0, t, 2048):
            runner.step([StepEntry(r, ids[r][at:min(t, at + 2048)], [])])
    assert calls == {"added": 0, "scaled": 0}, "portions of prompts take the kernels for many rows"
    want = [plain.logits(x, cfg_json, w) for x in ids]
    for i in range(steps):
        got = runner.step([StepEntry(r, [ids[r][t + i]], [0]) for r, t in enumerate(lengths)]).cpu()
        for r, t in enumerate(lengths):
            err = float((got[r] - want[r][t + i]).abs().max())
            assert err <= tolerance("bfloat16", want[r][t + i]), f"step {i}, request {r}: {err}"
    assert bool(runner._graphs) == use_graphs
    assert calls["added"] >= cfg.num_layers and calls["scaled"] == calls["added"], \
        "the decode steps did not take the products that add into the stream"
    runner.manager.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_layers_launched_from_a_recorded_layer_give_the_same_bits(dtype):
    """Steps that are not replayed from a graph record the launches of one layer of a kind
    and launch the others from the list.  Against the same steps with every layer run as
    written: equal bits of every logit, step after step (portions of two requests beside a
    decode token, a whole prompt, decode steps of few rows with their fused products, a
    step of 70 tokens), and the same cache afterwards; and the list was in fact used."""
    from tokamak_amd.engine import layer_replay
    from tokamak_amd.engine.runner import ModelRunner, StepEntry

    cfg, cfg_json, plan, source, w = shaped("qwen3-0.6b", on_gpu=True, num_layers=5, vocab_size=2048,
                                            max_position_embeddings=1024)
    ids = [random_ids(cfg.vocab_size, 400, 70 + i) for i in range(4)]
    launched = []
    launch = layer_replay.LayerRecording.launch

    def run(replay):
        runner = ModelRunner(plan, source, dtype=dtype, page_size=16, kv_pool_tokens=2048, max_requests=4, use_graphs=False)
        runner.model.replay_layers = replay
        out = []
        out.append(runner.step([StepEntry(0, ids[0][:150], [149])]))
        out.append(runner.step([StepEntry(1, ids[1][:90], [0, 89]), StepEntry(0, ids[0][150:151], [0]),
                                StepEntry(2, ids[2][:37], [])]))
        out.append(runner.step([StepEntry(r, ids[r][n:n + 1], [0]) for r, n in ((0, 151), (1, 90), (2, 37))]))
        out.append(runner.step([StepEntry(3, ids[3][:70], [69])]))
        out.append(runner.step([StepEntry(2, ids[2][38:40], [1]), StepEntry(3, ids[3][70:73], [2])]))
        torch.cuda.synchronize()
        cache = [a.clone() for slot in sorted(runner.storage._slots) for a in runner.storage.slot(slot).arrays.values()]
        return [o.cpu() for o in out], cache

    packed = []

    def counted(self, tensors, then):
        launched.append(len(self.calls))
        packed.append(self.packed is not None and len(self.packed.expected) == len(self.calls))
        return launch(self, tensors, then)

    plainly, cache_plain = run(False)
    try:
        layer_replay.LayerRecording.launch = counted
        replayed, cache_replayed = run(True)
        # ... and once more with the lists issued call by call from Python (what a recording falls
        # back to when an entry point has no slot form)
        layer_replay.LayerRecording.launch = lambda self, tensors, then: (
            setattr(self, "pack_tried", True), launch(self, tensors, then))[1]
        by_call, cache_by_call = run(True)
    finally:
        layer_replay.LayerRecording.launch = launch
    assert len(launched) == 5 * (cfg.num_layers - 2), "three of five layers of every step are launched from the list"
    assert min(launched) >= 5
    # a list is issued call by call at its first replay and packed behind it: of the three replayed
    # layers of a step the second and third go out in one foreign call each (csrc/replay.hip)
    assert packed == [False, True, True] * 5, packed
    for a, b in zip(replayed, by_call):
        assert torch.equal(a, b)
    for a, b in zip(cache_replayed, cache_by_call):
        assert torch.equal(a, b)
    for step, (a, b) in enumerate(zip(plainly, replayed)):
        assert torch.equal(a, b), f"step {step}: {float((a - b).abs().max())}"
    for a, b in zip(cache_plain, cache_replayed):
        assert torch.equal(a, b)
    want = plain.logits(ids[0][:152], cfg_json, w)
    err = float((replayed[2][0] - want[151]).abs().max())
    assert err <= tolerance(dtype, want[151]), err
